"""GPU parity: every stage of the HIP path against the CPU oracle, through the C ABI
(ctypes) exactly as a caller would reach it.  Integer, int8 and index outputs must be
bit-exact; bf16 outputs of the canonical-order kernels are bit-exact as well, and the
fused-scale variants must stay within max-abs <= 1e-2 * max|ref| and mean-rel <= 2e-3."""
import math
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

BS_ALL = (16, 32, 64, 128)


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib

    _lib.lib()  # a missing HIP library must fail the run, not skip it
    return torch.device("cuda:0")


def within_tolerance(out, ref):
    o, r = out.float().cpu(), ref.float().cpu()
    err = (o - r).abs()
    return err.max().item() <= 1e-2 * r.abs().max().item() and \
        (err.sum() / r.abs().sum().clamp(min=1e-30)).item() <= 2e-3


# ------------------------------------------------------------------ alignment --

@pytest.mark.parametrize("S,E,bs", [(1, 8, 16), (2, 64, 16), (7, 4, 16), (128, 8, 16), (512, 256, 16),
                                    (1000, 33, 32), (4096, 128, 64), (8191, 5, 128), (32768, 256, 64),
                                    (65536, 256, 128), (131072, 256, 16), (3000, 1000, 16)])
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_align_bit_exact(dev, oracle, S, E, bs, idt):
    from lightop_amd.moe import moe_align_block_size

    say(f"align S={S} E={E} bs={bs} {idt}")
    g = torch.Generator().manual_seed(S + E)
    ids = torch.randint(0, E, (S,), generator=g, dtype=torch.int32)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
    s, e, p = moe_align_block_size(ids.to(idt).to(dev).view(-1, 1), bs, E)
    torch.cuda.synchronize()
    assert torch.equal(p.cpu(), rp)
    assert torch.equal(s.cpu(), rs), "sorted_token_ids differ"
    assert torch.equal(e.cpu(), re), "expert_ids differ"


@pytest.mark.parametrize("ignore", [False, True])
@pytest.mark.parametrize("tokens", [333, 4099])  # one workgroup / many workgroups
def test_align_expert_map(dev, oracle, ignore, tokens):
    from lightop_amd.moe import moe_align_block_size

    say(f"align expert_map ignore={ignore} tokens={tokens}")
    g = torch.Generator().manual_seed(11)
    E = 256
    ids = torch.randint(0, E, (tokens, 8), generator=g, dtype=torch.int32)
    emap = torch.full((E,), -1, dtype=torch.int32)
    emap[64:96] = torch.arange(32, dtype=torch.int32)
    rs, re, rp = oracle.moe_align_block_size(ids, 16, E, expert_map=emap, ignore_invalid_experts=ignore)
    s, e, p = moe_align_block_size(ids.to(dev), 16, E, expert_map=emap.to(dev), ignore_invalid_experts=ignore)
    torch.cuda.synchronize()
    assert torch.equal(p.cpu(), rp) and torch.equal(s.cpu(), rs) and torch.equal(e.cpu(), re)


def test_align_skewed_and_docstring(dev, oracle):
    from lightop_amd.moe import moe_align_block_size

    say("align docstring + all-one-expert")
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    s, e, p = moe_align_block_size(ids.to(dev), 4, 5)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert p.item() == 16 and e[:4].tolist() == [1, 2, 3, 4]
    ids = torch.full((5000,), 3, dtype=torch.int32)
    rs, re, rp = oracle.moe_align_block_size(ids, 64, 8)
    s, e, p = moe_align_block_size(ids.to(dev).view(-1, 1), 64, 8)
    assert torch.equal(s.cpu(), rs) and torch.equal(e.cpu(), re) and torch.equal(p.cpu(), rp)


def test_align_out_variant_and_errors(dev, oracle):
    from lightop_amd.moe import moe_align_block_size_out

    say("align out variant")
    ids = torch.randint(0, 16, (64, 2), dtype=torch.int32)
    cap, nb = oracle.align_buffer_sizes(128, 16, 16)
    s = torch.empty(cap, dtype=torch.int32, device=dev)
    e = torch.empty(nb, dtype=torch.int32, device=dev)
    p = torch.empty(1, dtype=torch.int32, device=dev)
    moe_align_block_size_out(ids.to(dev), 16, 16, s, e, p)
    rs, re, rp = oracle.moe_align_block_size(ids, 16, 16)
    assert torch.equal(s.cpu(), rs) and torch.equal(e.cpu(), re) and torch.equal(p.cpu(), rp)
    with pytest.raises(RuntimeError):
        moe_align_block_size_out(ids.to(dev), 16, 16, s[:10], e, p)


@pytest.mark.parametrize("M,k,E", [(40, 4, 16), (3000, 8, 128)])  # one workgroup / many workgroups
@pytest.mark.parametrize("is_ep", [False, True])
def test_align_num_local_tokens_and_mask_output(dev, oracle, M, k, E, is_ep):
    """op.moe_align_block_size with its padded-batch and expert-parallel arguments."""
    from lightop_amd import op

    g = torch.Generator().manual_seed(M + k)
    ids = torch.randint(0, E, (M, k), generator=g, dtype=torch.int32)
    emap = torch.full((E,), -1, dtype=torch.int32)
    emap[: E // 2] = torch.arange(E // 2, dtype=torch.int32)
    bs = 16
    cap, nb = oracle.align_buffer_sizes(M * k, E, bs)
    for n in (0, 1, M // 3, M):
        say(f"align padded batch M={M} k={k} local={n} is_ep={is_ep}")
        s = torch.full((cap,), -7, dtype=torch.int32, device=dev)
        e = torch.full((nb,), -7, dtype=torch.int32, device=dev)
        p = torch.full((1,), -7, dtype=torch.int32, device=dev)
        mask = torch.ones(M * k, dtype=torch.bool, device=dev)
        nlt = torch.tensor([n], dtype=torch.int32, device=dev)
        op.moe_align_block_size(ids.to(dev), E, bs, s, e, p, emap.to(dev), mask, nlt, is_ep)
        torch.cuda.synchronize()
        rs, re, rp = oracle.moe_align_block_size(ids, bs, E, expert_map=emap, ignore_invalid_experts=is_ep,
                                                 num_local_tokens=n)
        assert torch.equal(p.cpu(), rp) and torch.equal(s.cpu(), rs) and torch.equal(e.cpu(), re)
        assert torch.equal(mask.cpu(), oracle.align_slot_mask(ids, emap, n))


def test_moe_sum_num_local_tokens(dev, oracle):
    from lightop_amd.moe import moe_sum

    say("moe_sum padded batch")
    g = torch.Generator().manual_seed(12)
    x = torch.randn(50, 4, 256, generator=g).to(torch.bfloat16)
    bias = torch.randn(50, 256, generator=g).to(torch.bfloat16)
    for n in (0, 1, 17, 50, 80):
        for b in (None, bias):
            prev = torch.full((50, 256), 3.0, dtype=torch.bfloat16)
            out = prev.clone().to(dev)
            moe_sum(x.to(dev), out, None if b is None else b.to(dev),
                    num_local_tokens=torch.tensor([n], dtype=torch.int32, device=dev), factor=1.5)
            torch.cuda.synchronize()
            ref = oracle.moe_sum(x, b, 1.5, num_local_tokens=n, out=prev)
            assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16)), f"n={n}"


# ---------------------------------------------------------------- group quant --

@pytest.mark.parametrize("rows,cols", [(1, 128), (1, 7168), (3, 2048), (64, 1024), (257, 768), (4096, 2048)])
def test_group_quant_bit_exact(dev, oracle, rows, cols):
    from lightop_amd.quant import per_token_group_quant_int8

    say(f"quant {rows}x{cols}")
    g = torch.Generator().manual_seed(rows * 13 + cols)
    x = (torch.randn(rows, cols, generator=g) * torch.rand(rows, 1, generator=g) * 8).to(torch.bfloat16)
    x[0, :128] = 0  # an all-zero group
    if rows > 1:
        x[1, 5] = 300.0
    rq, rs = oracle.per_token_group_quant_int8(x)
    q, s = per_token_group_quant_int8(x.to(dev), 128)
    torch.cuda.synchronize()
    assert q.dtype == torch.int8 and s.dtype == torch.float32 and s.shape == (rows, cols // 128)
    assert torch.equal(s.cpu(), rs), "scales differ"
    assert torch.equal(q.cpu(), rq), "int8 values differ"


def test_group_quant_truncation_cases(dev):
    from lightop_amd.quant import per_token_group_quant_int8

    say("quant truncation cases")
    row = [127.0, 1.5, -1.5, 2.5, -2.5, 0.75, -0.75, 126.5] + [0.0] * 120
    q, s = per_token_group_quant_int8(torch.tensor([row]).to(torch.bfloat16).to(dev), 128)
    assert s.item() == 1.0 and q[0, :8].tolist() == [127, 1, -1, 2, -2, 0, 0, 126]
    with pytest.raises(AssertionError):
        per_token_group_quant_int8(torch.zeros(2, 100, dtype=torch.bfloat16, device=dev), 128)


# --------------------------------------------------------------- SiLU * mul ----

def test_silu_and_mul_every_bf16(dev, oracle):
    from lightop_amd.moe import silu_and_mul

    say("silu_and_mul over all bf16 gates")
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(512, 128)
    finite = torch.isfinite(gate.float())
    gate = torch.where(finite, gate, torch.zeros_like(gate))
    g = torch.Generator().manual_seed(4)
    up = torch.randn(512, 128, generator=g).to(torch.bfloat16)
    c1 = torch.cat([gate, up], dim=1).contiguous()
    ref = oracle.silu_and_mul(c1)
    out = torch.empty(512, 128, dtype=torch.bfloat16, device=dev)
    silu_and_mul(out, c1.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


# ------------------------------------------------------------------ moe_sum ----

@pytest.mark.parametrize("M,k,H", [(1, 8, 7168), (5, 2, 1024), (64, 8, 2048), (33, 1, 256), (300, 6, 4096)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_moe_sum_bit_exact(dev, oracle, M, k, H, with_bias):
    from lightop_amd.moe import moe_sum

    say(f"moe_sum M={M} k={k} H={H} bias={with_bias}")
    g = torch.Generator().manual_seed(M + k + H)
    x = torch.randn(M, k, H, generator=g).to(torch.bfloat16)
    b = torch.randn(M, H, generator=g).to(torch.bfloat16) if with_bias else None
    ref = oracle.moe_sum(x, bias=b, factor=2.5)
    out = torch.empty(M, H, dtype=torch.bfloat16, device=dev)
    moe_sum(x.to(dev), out, bias=None if b is None else b.to(dev), factor=2.5)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_moe_sum_expert_mask(dev, oracle):
    """Masked slots are skipped: same result as summing zeros in their place."""
    from lightop_amd.moe import moe_sum

    say("moe_sum expert_mask")
    g = torch.Generator().manual_seed(8)
    M, k, H = 37, 8, 1024
    x = torch.randn(M, k, H, generator=g).to(torch.bfloat16)
    mask = torch.rand(M, k, generator=g) > 0.6
    mask[3] = False  # a token with no local expert
    ref = oracle.moe_sum(torch.where(mask[..., None], x, torch.zeros_like(x)), factor=2.5)
    garbage = torch.where(mask[..., None], x, torch.full_like(x, float("nan")))
    out = torch.empty(M, H, dtype=torch.bfloat16, device=dev)
    moe_sum(garbage.to(dev), out, expert_mask=mask.reshape(-1).to(dev), factor=2.5)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


# --------------------------------------------------------------------- GEMM ----

# The two scale orders the CPU checker restates bit for bit: the library's default, acc = fma(f32(d) * a_s, b_s, acc),
# and the order without fp fusion, acc = acc + (f32(d) * a_s) * b_s (flag LO_GEMM_SEPARATE_ORDER).
ORDERS = ["contract", "separate"]


def order_flag(order):
    from lightop_amd import _lib

    return _lib.LO_GEMM_SEPARATE_ORDER if order == "separate" else 0


def gemm_case(seed, M, k, E, Eg, N, K, small_values=False):
    g = torch.Generator().manual_seed(seed)
    lo, hi = (-7, 8) if small_values else (-127, 128)
    Aq = torch.randint(lo, hi, (M, K), generator=g, dtype=torch.int8)
    W = torch.randint(lo, hi, (E, N, K), generator=g, dtype=torch.int8)
    if small_values:
        As = torch.ones(M, K // 128)
        Ws = torch.ones(E, (N + 127) // 128, K // 128)
    else:
        As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
        Ws = torch.exp(torch.randn(E, (N + 127) // 128, K // 128, generator=g) * 0.3 + math.log(1e-3))
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = None
    if Eg != E:
        emap = torch.full((Eg,), -1, dtype=torch.int32)
        emap[:E] = torch.arange(E, dtype=torch.int32)
    return Aq, As, W, Ws, ids, tw, emap


@pytest.mark.parametrize("M,k,E,Eg,N,K", [(1, 2, 4, 4, 64, 128), (5, 2, 4, 4, 256, 512), (40, 4, 8, 8, 320, 1024),
                                          (64, 2, 8, 8, 1024, 1024), (100, 8, 4, 16, 512, 768),
                                          (300, 2, 3, 3, 128, 2048)])
@pytest.mark.parametrize("bs", BS_ALL)
@pytest.mark.parametrize("order", ORDERS)
def test_gemm_bit_exact(dev, oracle, M, k, E, Eg, N, K, bs, order):
    from lightop_amd.moe import invoke_fused_moe_kernel_int8, moe_align_block_size, preshuffle_moe_weight

    say(f"gemm M={M} k={k} E={E}/{Eg} N={N} K={K} bs={bs} order={order}")
    Aq, As, W, Ws, ids, tw, emap = gemm_case(M + N + bs, M, k, E, Eg, N, K)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    S = M * k
    # the 64- and 128-token tiles have two implementations: LDS-tiled (default) and weight-streaming
    impls = (0, 2) if bs >= 64 else (0,)
    Wd = W.to(dev)
    Wsh = preshuffle_moe_weight(Wd)
    for mul in (False, True):
        with oracle.scale_order(order):
            ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, S, bs)
        for force_streaming in impls:
            for Wx in (Wd, Wsh):  # row-major and load-time pre-shuffled weights
                C = torch.full((M, k, N), 7.0, dtype=torch.bfloat16, device=dev)
                s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
                invoke_fused_moe_kernel_int8(Aq.to(dev), Wx, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p,
                                             mul, k, {"BLOCK_SIZE_M": bs}, flags=force_streaming | order_flag(order))
                torch.cuda.synchronize()
                assert torch.equal(C.view(S, N).cpu().view(torch.int16), ref.view(torch.int16)), \
                    f"mul_routed={mul} flags={force_streaming} preshuffled={Wx is Wsh}"
    # fused-scale variant: same integers, fp32 rounding differs in the last place only
    C2 = torch.empty((M, k, N), dtype=torch.bfloat16, device=dev)
    invoke_fused_moe_kernel_int8(Aq.to(dev), Wsh, C2, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p,
                                 True, k, {"BLOCK_SIZE_M": bs}, fused_scale=True)
    torch.cuda.synchronize()
    assert within_tolerance(C2.view(S, N), ref)
    differs = (C2.view(S, N).cpu().view(torch.int16) != ref.view(torch.int16)).float().mean().item()
    assert differs < 0.02, differs


@pytest.mark.parametrize("bs", BS_ALL)
def test_gemm_int32_accumulators_exact(dev, oracle, bs):
    """Unit scales and small integers: the bf16 output is then the exactly rounded integer
    dot product, in any summation order, for both scale modes."""
    from lightop_amd.moe import invoke_fused_moe_kernel_int8, moe_align_block_size

    say(f"gemm integer exactness bs={bs}")
    M, k, E, N, K = 70, 2, 4, 256, 7168
    Aq, As, W, Ws, ids, tw, emap = gemm_case(99 + bs, M, k, E, E, N, K, small_values=True)
    exact = torch.einsum("mk,enk->men", Aq.double(), W.double())  # [M, E, N], exact in float64
    s, e, p = moe_align_block_size(ids.to(dev), bs, E)
    for fused in (False, True):
        C = torch.empty((M, k, N), dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), W.to(dev), C, As.to(dev), Ws.to(dev), None, s, e, p,
                                     False, k, {"BLOCK_SIZE_M": bs}, fused_scale=fused)
        torch.cuda.synchronize()
        want = torch.stack([exact[m, ids[m].long()] for m in range(M)])  # [M, k, N]
        assert torch.equal(C.cpu(), want.float().to(torch.bfloat16)), f"fused_scale={fused}"


@pytest.mark.parametrize("M,k,E,Eg,I,K", [(1, 2, 4, 4, 128, 256), (9, 2, 4, 4, 256, 512), (64, 2, 8, 8, 512, 1024),
                                          (50, 8, 4, 16, 256, 768), (200, 4, 6, 6, 384, 1024)])
@pytest.mark.parametrize("bs", BS_ALL)
@pytest.mark.parametrize("order", ORDERS)
def test_gemm1_silu_quant_bit_exact(dev, oracle, M, k, E, Eg, I, K, bs, order):
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_weight

    say(f"gemm1+silu+quant M={M} k={k} E={E}/{Eg} I={I} K={K} bs={bs} order={order}")
    Aq, As, W, Ws, ids, tw, emap = gemm_case(M + I + bs + 1, M, k, E, Eg, 2 * I, K)
    Ws = Ws * 30  # bring the gate into the range where SiLU is neither 0 nor identity
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    S = M * k
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    impls = (0, 2) if bs >= 64 else (0,)
    for mul in (False, True):
        with oracle.scale_order(order):
            c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, S, bs)
        rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
        for force_streaming in impls:
            for Wx in (W.to(dev), preshuffle_moe_weight(W.to(dev))):
                q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wx, As.to(dev), Ws.to(dev), tw.to(dev),
                                                          s, e, p, mul, k, S, {"BLOCK_SIZE_M": bs},
                                                          flags=force_streaming | order_flag(order))
                torch.cuda.synchronize()
                local = torch.ones(S, dtype=torch.bool) if emap is None else emap.long()[ids.reshape(-1).long()] >= 0
                what = f"mul_routed={mul}, flags={force_streaming}, preshuffled={hasattr(Wx, 'lo_preshuffled')}"
                assert torch.equal(sc.cpu()[local], rsc[local]), f"scales differ ({what})"
                assert torch.equal(q.cpu()[local], rq[local]), f"int8 activations differ ({what})"


@pytest.mark.parametrize("bs", [16, 64, 128])
def test_gemm1_epilogue_every_finite_bf16_gate(dev, oracle, bs):
    """Every bf16 value below 1e18 in magnitude as the gate of the fused epilogue (SiLU table, its LDS band and the
    closed forms outside the band): token t's group scale is the t-th bf16 pattern and the single
    non-zero product of its row is 1, so gate = up = that value."""
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size

    say(f"gemm1 epilogue over all bf16 gates bs={bs}")
    pat = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    # gate * up must stay finite: with an infinite activation the group scale is inf, the quotient
    # NaN and its int8 image undefined (in the reference as well)
    pat = pat[torch.isfinite(pat) & (pat.abs() < 1e18)]
    M, I, K = pat.numel(), 128, 128
    Aq = torch.zeros(M, K, dtype=torch.int8)
    Aq[:, 0] = 1
    W = torch.zeros(1, 2 * I, K, dtype=torch.int8)
    W[0, :, 0] = 1
    As = pat.reshape(M, 1).contiguous()
    Ws = torch.ones(1, 2, 1)
    ids = torch.zeros(M, 1, dtype=torch.int32)
    tw = torch.ones(M, 1)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, 1)
    c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, 1, M, bs)
    assert torch.equal(c1[:, 0].float(), pat)  # the construction works: gate == pattern
    rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
    s, e, p = moe_align_block_size(ids.to(dev), bs, 1)
    from lightop_amd.moe import preshuffle_moe_weight
    for Wx in (W.to(dev), preshuffle_moe_weight(W.to(dev))):  # the two layouts have kernels of their own
        for fused_scale in (False, True):  # unit weight scales: both orders give the same values
            q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wx, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p,
                                                      False, 1, M, {"BLOCK_SIZE_M": bs}, fused_scale=fused_scale)
            torch.cuda.synchronize()
            assert torch.equal(sc.cpu(), rsc) and torch.equal(q.cpu(), rq)


@pytest.mark.parametrize("bs", [64, 128])
def test_gemm1_epilogue_nan_and_inf_gates(dev, oracle, bs):
    """Gates that are NaN or infinite leave the fast lookup: rows that hold one, next to ordinary
    rows in the same wavefront.  The activation's scale is then inf or NaN; what is pinned is that
    the ordinary rows are untouched and the special rows agree with the oracle where it is finite."""
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_weight

    say(f"gemm1 epilogue, NaN and inf gates bs={bs}")
    M, I, K = 200, 128, 128
    g = torch.Generator().manual_seed(3)
    Aq = torch.zeros(M, K, dtype=torch.int8)
    Aq[:, 0] = 1
    W = torch.zeros(1, 2 * I, K, dtype=torch.int8)
    W[0, :, 0] = 1
    vals = torch.randn(M, generator=g) * 3
    vals[5], vals[70], vals[71], vals[150] = float("inf"), float("-inf"), float("nan"), float("-inf")
    As = vals.reshape(M, 1).contiguous()
    Ws = torch.ones(1, 2, 1)
    ids = torch.zeros(M, 1, dtype=torch.int32)
    tw = torch.ones(M, 1)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, 1)
    c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, 1, M, bs)
    rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
    s, e, p = moe_align_block_size(ids.to(dev), bs, 1)
    ordinary = torch.isfinite(vals)
    for Wx in (W.to(dev), preshuffle_moe_weight(W.to(dev))):
        q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wx, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p,
                                                  False, 1, M, {"BLOCK_SIZE_M": bs}, fused_scale=False)
        torch.cuda.synchronize()
        assert torch.equal(sc.cpu()[ordinary], rsc[ordinary]) and torch.equal(q.cpu()[ordinary], rq[ordinary])
        special = ~ordinary
        same_class = (torch.isnan(sc.cpu()[special]) == torch.isnan(rsc[special])) & \
                     (torch.isinf(sc.cpu()[special]) == torch.isinf(rsc[special]))
        assert same_class.all()


@pytest.mark.parametrize("bs", [64, 128])
def test_gemm_sorted_ids_with_gaps(dev, oracle, bs):
    """A caller's own sorted ids need not keep a block's valid slots at its front: padding entries
    anywhere inside a block (here: a random permutation of every block) must give the same rows."""
    from lightop_amd.moe import (invoke_fused_moe_gemm1_silu_quant, invoke_fused_moe_kernel_int8,
                                 preshuffle_moe_weight)

    say(f"sorted ids with gaps bs={bs}")
    M, k, E, I, K = 150, 2, 3, 128, 384
    Aq, As, W, Ws, ids, tw, _ = gemm_case(11 + bs, M, k, E, E, 2 * I, K)
    Ws = Ws * 30
    rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
    g = torch.Generator().manual_seed(bs)
    P = int(rp)
    rs = rs.clone()
    for b in range(P // bs):
        rs[b * bs:(b + 1) * bs] = rs[b * bs:(b + 1) * bs][torch.randperm(bs, generator=g)]
    S = M * k
    ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, True, k, S, bs)
    c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, k, S, bs)
    rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
    s, e, p = rs.to(dev), re.to(dev), rp.to(dev)
    for Wx in (W.to(dev), preshuffle_moe_weight(W.to(dev))):
        C = torch.full((M, k, 2 * I), 7.0, dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), Wx, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, True, k,
                                     {"BLOCK_SIZE_M": bs}, fused_scale=False)
        q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wx, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False,
                                                  k, S, {"BLOCK_SIZE_M": bs}, fused_scale=False)
        torch.cuda.synchronize()
        assert torch.equal(C.view(S, -1).cpu().view(torch.int16), ref.view(torch.int16))
        assert torch.equal(sc.cpu(), rsc) and torch.equal(q.cpu(), rq)


@pytest.mark.parametrize("count,K", [(c, 384) for c in (1, 31, 32, 33, 64, 65, 96, 97, 127, 128, 129, 200)] +
                         [(c, k) for k in (128, 256, 1024) for c in (40, 128, 250)])
@pytest.mark.parametrize("order", ORDERS)
def test_gemm_128_token_blocks_fill_levels(dev, oracle, count, K, order):
    """128-token blocks holding 1 ... 128 valid tokens: the K loop of the 128-token kernel comes in
    variants by the number of 32-token pieces in use, and padded pieces are skipped.  One, two and
    eight K blocks as well: the full-tile variant reads a K block's first operands during the
    previous one and keeps the token scales two K blocks ahead."""
    from lightop_amd.moe import (invoke_fused_moe_gemm1_silu_quant, invoke_fused_moe_kernel_int8,
                                 moe_align_block_size, preshuffle_moe_weight)

    say(f"128-token blocks, {count} tokens on expert 0, K = {K}, order={order}")
    bs, E, I = 128, 2, 128
    M = count + 3
    Aq, As, W, Ws, _, tw, _ = gemm_case(count, M, 1, E, E, 2 * I, K)
    Ws = Ws * 30
    ids = torch.ones(M, 1, dtype=torch.int32)
    ids[torch.randperm(M, generator=torch.Generator().manual_seed(count))[:count]] = 0
    rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
    s, e, p = moe_align_block_size(ids.to(dev), bs, E)
    Wsh = preshuffle_moe_weight(W.to(dev))
    with oracle.scale_order(order):
        ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, True, 1, M, bs)
        c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, 1, M, bs)
    C = torch.full((M, 1, 2 * I), 7.0, dtype=torch.bfloat16, device=dev)
    invoke_fused_moe_kernel_int8(Aq.to(dev), Wsh, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, True, 1,
                                 {"BLOCK_SIZE_M": bs}, flags=order_flag(order))
    torch.cuda.synchronize()
    assert torch.equal(C.view(M, -1).cpu().view(torch.int16), ref.view(torch.int16))
    rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
    q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wsh, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False, 1,
                                              M, {"BLOCK_SIZE_M": bs}, flags=order_flag(order))
    torch.cuda.synchronize()
    assert torch.equal(sc.cpu(), rsc) and torch.equal(q.cpu(), rq)


def test_preshuffle_layout(dev):
    from lightop_amd.moe import preshuffle_moe_weight

    say("preshuffle layout")
    E, N, K = 3, 48, 384
    w = torch.arange(E * N * K, dtype=torch.int64).remainder(251).sub(125).to(torch.int8).view(E, N, K)
    got = preshuffle_moe_weight(w.to(dev)).cpu()
    # [E, N/16, 16 rows, K/128, 8 chunks, 16 B] -> [E, K/128, N/16, 8 chunks, 16 rows, 16 B]
    want = w.view(E, N // 16, 16, K // 128, 8, 16).permute(0, 3, 1, 4, 2, 5).contiguous().view(E, N, K)
    assert torch.equal(got, want)


# ---------------------------------------------------------------- whole path ---

def run_fused(dev, layer, M, seed, bs=0, flags=0, shared=False, on_input=False, inplace=False, preshuffle=False):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, preshuffle_moe_weight

    w1, w2, w1s, w2s = wl.make_weights(layer, seed=seed)
    x, tw, ids = wl.make_inputs(layer, M, seed=seed)
    emap = wl.expert_map_for(layer)
    g = torch.Generator().manual_seed(seed + 5)
    sh = torch.randn(M, layer.H, generator=g).to(torch.bfloat16) if shared else None
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    xd = x.to(dev)
    w1d, w2d = w1.to(dev), w2.to(dev)
    if preshuffle:
        w1d, w2d = preshuffle_moe_weight(w1d), preshuffle_moe_weight(w2d)
    out = fused_experts_impl_int8(
        xd, w1d, w2d, tw.to(dev), ids.to(dev), cache13, inplace=inplace,
        apply_router_weight_on_input=on_input, use_int8_w8a8=True, global_num_experts=layer.E_global,
        expert_map=None if emap is None else emap.to(dev), w1_scale=w1s.to(dev), w2_scale=w2s.to(dev),
        block_shape=[128, 128], routed_scaling_factor=1.0 if not shared else 2.5,
        shared_output=None if sh is None else sh.to(dev), lightop_amd_block_size_m=bs, lightop_amd_flags=flags)
    torch.cuda.synchronize()
    if inplace:
        assert out.data_ptr() == xd.data_ptr()
    return (x, w1, w2, w1s, w2s, tw, ids, emap, sh), out.cpu()


@pytest.mark.parametrize("bs", BS_ALL)
@pytest.mark.parametrize("preshuffle", [False, True])
@pytest.mark.parametrize("order", ORDERS)
def test_fused_experts_tiny_config_bit_exact(dev, oracle, bs, preshuffle, order):
    """The tiny benchmark configuration: E=8, top-2, H=1024, I=512, M=64, seed 0."""
    from lightop_amd import workloads as wl

    say(f"fused tiny bs={bs} preshuffle={preshuffle} order={order}")
    (x, w1, w2, w1s, w2s, tw, ids, emap, sh), out = run_fused(dev, wl.TINY, 64, 0, bs=bs, preshuffle=preshuffle,
                                                              flags=order_flag(order))
    with oracle.scale_order(order):
        ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, bs)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 3, 16, 77])
@pytest.mark.parametrize("variant", ["plain", "shared", "on_input", "inplace"])
def test_fused_experts_ep_share_bit_exact(dev, oracle, M, variant):
    from lightop_amd import workloads as wl

    say(f"fused ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid",
                        n_group=8, topk_group=4, routed_scaling=2.5)
    kw = dict(shared=variant == "shared", on_input=variant == "on_input", inplace=variant == "inplace")
    (x, w1, w2, w1s, w2s, tw, ids, emap, sh), out = run_fused(dev, layer, M, 3, bs=16, **kw)
    ref = oracle.fused_experts_block_int8(
        x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
        apply_router_weight_on_input=kw["on_input"], routed_scaling_factor=2.5 if kw["shared"] else 1.0,
        shared_output=sh)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_fused_experts_default_tile_and_fused_scale(dev, oracle):
    """Block size from the tile table: the default arithmetic is bit-exact, the optional fused-scale
    order within the tolerance."""
    from lightop_amd import _lib, workloads as wl

    say("fused default tile + fused-scale tolerance")
    layer = wl.MoeLayer("q", E=16, E_global=16, top_k=4, H=512, I=256, routing="softmax")
    for pre in (False, True):
        (x, w1, w2, w1s, w2s, tw, ids, emap, sh), out = run_fused(dev, layer, 200, 1, preshuffle=pre)
        ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 64)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"default order, preshuffle={pre}"
        _, out_s = run_fused(dev, layer, 200, 1, flags=_lib.LO_GEMM_SEPARATE_ORDER, preshuffle=pre)
        with oracle.scale_order("separate"):
            ref_s = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 64)
        assert torch.equal(out_s.view(torch.int16), ref_s.view(torch.int16)), f"separate order, preshuffle={pre}"
        _, out_f = run_fused(dev, layer, 200, 1, flags=_lib.LO_GEMM_FUSED_SCALE, preshuffle=pre)
        assert within_tolerance(out_f, ref)


@pytest.mark.parametrize("bs", BS_ALL)
def test_expert_map_entry_outside_the_weights_gives_zero_rows(dev, oracle, bs):
    """A malformed expert_map (a local id >= the number of experts held) must not read past the
    weights nor leave garbage in the sum: such slots contribute zero, exactly as if the entry were -1."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, preshuffle_moe_weight

    say(f"expert_map entry >= E, bs={bs}")
    layer = wl.MoeLayer("oob", E=4, E_global=8, top_k=2, H=256, I=128, routing="softmax")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=2)
    M = 150
    x, tw, ids = wl.make_inputs(layer, M, seed=2)
    bad = torch.tensor([0, 1, 2, 3, 4, 9, -1, 1000], dtype=torch.int32)     # 4, 9, 1000: outside w1 / w2
    good = torch.tensor([0, 1, 2, 3, -1, -1, -1, -1], dtype=torch.int32)
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, bs, global_num_experts=8, expert_map=good)
    for pre in (False, True):
        w1d, w2d = w1.to(dev), w2.to(dev)
        if pre:
            w1d, w2d = preshuffle_moe_weight(w1d), preshuffle_moe_weight(w2d)
        cache13 = torch.full((M * 2 * 256,), float("nan"), dtype=torch.bfloat16, device=dev)
        out = fused_experts_impl_int8(x.to(dev), w1d, w2d, tw.to(dev), ids.to(dev), cache13, use_int8_w8a8=True,
                                      global_num_experts=8, expert_map=bad.to(dev), w1_scale=w1s.to(dev),
                                      w2_scale=w2s.to(dev), block_shape=[128, 128], lightop_amd_block_size_m=bs)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16)), f"preshuffle={pre}"


def test_fused_experts_rejects_unsupported(dev):
    from lightop_amd.moe import fused_experts_impl_int8

    x = torch.zeros(2, 256, dtype=torch.bfloat16, device=dev)
    w1 = torch.zeros(2, 256, 256, dtype=torch.int8, device=dev)
    w2 = torch.zeros(2, 256, 128, dtype=torch.int8, device=dev)
    tw = torch.ones(2, 1, device=dev)
    ids = torch.zeros(2, 1, dtype=torch.int32, device=dev)
    c = torch.empty(2 * 256, dtype=torch.bfloat16, device=dev)
    s1 = torch.ones(2, 2, 2, device=dev)
    s2 = torch.ones(2, 2, 1, device=dev)
    with pytest.raises(NotImplementedError):
        fused_experts_impl_int8(x, w1, w2, tw, ids, c, use_int8_w8a8=True, block_shape=[64, 64],
                                w1_scale=s1, w2_scale=s2)
    with pytest.raises(NotImplementedError):
        fused_experts_impl_int8(x, w1, w2, tw, ids, c, use_int8_w8a8=True, use_int8_w8a16=True,
                                block_shape=[128, 128], w1_scale=s1, w2_scale=s2)
    with pytest.raises(ValueError):
        fused_experts_impl_int8(x, w1, w2, tw, ids, c, use_int8_w8a8=True, block_shape=[128, 128],
                                activation="relu", w1_scale=s1, w2_scale=s2)
    with pytest.raises(AssertionError):
        fused_experts_impl_int8(x[:, :128], w1, w2, tw, ids, c, use_int8_w8a8=True, block_shape=[128, 128],
                                w1_scale=s1, w2_scale=s2)


def test_issue_rate_measurement_is_sane(dev):
    """lo_measure_mfma_issue_rate: positive rates below the published int8 peak, and the more vector instructions
    between the MFMAs the lower the rate; bad arguments are refused."""
    import ctypes

    from lightop_amd import _lib

    def rate(valu, random_operands, iters=4000):
        out = ctypes.c_double(0.0)
        rc = _lib.lib().lo_measure_mfma_issue_rate(valu, random_operands, iters,
                                                   ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
                                                   ctypes.byref(out))
        return rc, out.value

    rates = {}
    for valu in (0, 4, 6, 8):
        rc, v = rate(valu, 1)
        assert rc == 0 and 0.0 < v < 5.2e15
        rates[valu] = v
    assert rates[0] > rates[4] > rates[6] > rates[8]
    rc, zero = rate(0, 0)
    assert rc == 0 and zero >= 0.9 * rates[0]   # zeros toggle nothing: never slower than random bytes
    assert rate(5, 1)[0] == -1 and rate(6, 1, iters=0)[0] == -1   # LO_EINVAL
