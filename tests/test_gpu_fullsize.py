"""GPU parity at the benchmark's full sizes, where the oracle cannot run the whole problem.

Three kinds of checks:
  * size-independent properties of the routing alignment and the group quantisation;
  * two independent implementations (LDS-tiled and weight-streaming kernels, row-major
    and pre-shuffled weights) must agree bit for bit in both bit-exact scale orders;
  * tokens of a MoE layer are independent, so a random sample of tokens is pushed through
    the CPU oracle with only the experts those tokens use, and the sampled output rows, int8
    activations and scales of the full-size GPU run must equal the oracle's bit for bit in the
    library's default (contracted) order and in the order without fp fusion, or lie within the tolerance of
    the oracle in the optional fused-scale order.
"""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


_weights = {}


def layer_weights(layer, dev):
    """Full-size weights, generated on the device once per layer (row-major and pre-shuffled)."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    if layer.name not in _weights:
        _weights.clear()  # one layer resident at a time
        torch.cuda.empty_cache()
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
        _weights[layer.name] = (w1, w2, w1s, w2s, preshuffle_moe_weight(w1), preshuffle_moe_weight(w2))
    return _weights[layer.name]


def oracle_rows(oracle, layer, weights, x, tw, ids, emap, tokens, bs, intermediates=False):
    """Oracle output for the sampled tokens, using only the experts they touch.  With
    ``intermediates`` the oracle's dict of every stage (rows of a2q / a2s are slot t' * k + j of
    sampled token t') plus ``local``: which of those slots belong to an expert of this rank."""
    w1, w2, w1s, w2s = weights[:4]
    sub_ids = ids[tokens].cpu().long()
    local = sub_ids if emap is None else emap.cpu().long()[sub_ids]
    used = torch.unique(local[local >= 0])
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    # ids -> dense ids over the used experts; slots of other ranks' experts go to an id whose map entry is -1
    dense = torch.where(local >= 0, remap[local.clamp(min=0)], torch.full_like(local, used.numel()))
    dmap = torch.cat([torch.arange(used.numel(), dtype=torch.int32), torch.tensor([-1], dtype=torch.int32)])
    sel = used.to(w1.device)
    res = oracle.fused_experts_block_int8(
        x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(), tw[tokens].cpu(),
        dense.to(torch.int32), bs, global_num_experts=used.numel() + 1, expert_map=dmap,
        return_intermediates=intermediates)
    if intermediates:
        res["local"] = (local >= 0).reshape(-1)
    return res


def run_layer(layer, weights, x, tw, ids, emap, dev, bs, flags, preshuffled, workspace=None):
    from lightop_amd.moe import fused_experts_impl_int8

    w1, w2, w1s, w2s, w1p, w2p = weights
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_int8(
        x, w1p if preshuffled else w1, w2p if preshuffled else w2, tw, ids, cache13, use_int8_w8a8=True,
        global_num_experts=layer.E_global, expert_map=emap, w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128],
        lightop_amd_block_size_m=bs, lightop_amd_flags=flags, lightop_amd_workspace=workspace)
    torch.cuda.synchronize()
    return out


def run_with_intermediates(layer, weights, x, tw, ids, emap, dev, bs, flags, tokens):
    """Whole-path call on a caller-owned workspace; returns (out, a2q, a2s) with the int8 activations
    and their scales of the sampled tokens' slots, read back through the workspace offsets of the C ABI."""
    from lightop_amd.moe import fused_experts_workspace_bytes, fused_experts_workspace_views

    M, k = x.shape[0], layer.top_k
    ws = torch.empty(fused_experts_workspace_bytes(M, k, layer.H, layer.I, layer.E_global, 0), dtype=torch.uint8,
                     device=dev)
    out = run_layer(layer, weights, x, tw, ids, emap, dev, bs, flags, True, workspace=ws)
    v = fused_experts_workspace_views(ws, M, k, layer.H, layer.I, layer.E_global, bs)
    slots = (tokens[:, None] * k + torch.arange(k, device=dev)[None, :]).reshape(-1)
    return out, v["a2q"][slots].cpu(), v["a2s"][slots].cpu()


def within_tolerance(got, ref):
    """The path's tolerance against the oracle: max-abs <= 1e-2 * max|ref| and mean-rel <= 2e-3."""
    g, r = got.float(), ref.float()
    err = (g - r).abs()
    return bool(err.max() <= 1e-2 * r.abs().max()) and bool(err.sum() <= 2e-3 * r.abs().sum())


CASES = [  # (layer name, M, block sizes)
    ("qwen3-30b-a3b", 8192, (64, 128)),
    ("qwen3-30b-a3b", 512, (16, 32, 64)),
    ("deepseek-v3-ep8-share", 4096, (64, 128)),
    ("deepseek-v3-ep8-share", 64, (16,)),
    ("deepseek-v3-ep8-share", 1, (16,)),
]


@pytest.mark.parametrize("name,M,block_sizes", CASES)
def test_full_size_sampled_tokens_vs_oracle(dev, oracle, name, M, block_sizes):
    """The library's default arithmetic (acc = fma(f32(d) * a_s, b_s, acc) per K block, the one the benchmark times) at the
    benchmark's sizes: output rows, int8 activations between the GEMMs and their scales of sampled
    tokens equal the oracle's bit for bit, with both weight layouts and both kernel families; the
    optional fused-scale order stays within the path's tolerance of the oracle."""
    from lightop_amd import _lib, workloads as wl

    layer = wl.LAYERS[name]
    weights = layer_weights(layer, dev)
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    emap = wl.expert_map_for(layer, dev)
    g = torch.Generator().manual_seed(M)
    tokens = torch.randperm(M, generator=g)[: min(M, 6)].sort().values.to(dev)
    ref = oracle_rows(oracle, layer, weights, x, tw, ids, emap, tokens, 16, intermediates=True)
    loc = ref["local"]
    for bs in block_sizes:
        say(f"{name} M={M} bs={bs}")
        outs = []
        for pre in (True, False):
            for force in (0, _lib.LO_GEMM_FORCE_STREAMING):
                if force and bs < 64:
                    continue
                out = run_layer(layer, weights, x, tw, ids, emap, dev, bs, force, pre)
                got = out[tokens].cpu()
                assert torch.equal(got.view(torch.int16), ref["out"].view(torch.int16)), \
                    f"sampled rows differ from the oracle (bs={bs}, preshuffled={pre}, flags={force})"
                outs.append(out)
        for o in outs[1:]:  # and the implementations agree on every row, not only the sample
            assert torch.equal(o.view(torch.int16), outs[0].view(torch.int16))
        # the int8 activations that feed the second GEMM, in the default order: bit-exact
        out, a2q, a2s = run_with_intermediates(layer, weights, x, tw, ids, emap, dev, bs, 0, tokens)
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16))
        assert torch.equal(a2q[loc], ref["a2q"][loc]), f"a2q differs from the oracle in the default order (bs={bs})"
        assert torch.equal(a2s[loc].view(torch.int32), ref["a2s"][loc].view(torch.int32)), f"a2s differs (bs={bs})"
        # the order without fp fusion: bit-exact against the oracle in that order
        if bs == block_sizes[-1]:
            with oracle.scale_order("separate"):
                ref_s = oracle_rows(oracle, layer, weights, x, tw, ids, emap, tokens, 16, intermediates=True)
            out_s, a2q_s, a2s_s = run_with_intermediates(layer, weights, x, tw, ids, emap, dev, bs,
                                                         _lib.LO_GEMM_SEPARATE_ORDER, tokens)
            assert torch.equal(out_s[tokens].cpu().view(torch.int16), ref_s["out"].view(torch.int16)), \
                f"separate order: sampled rows differ from the oracle (bs={bs})"
            assert torch.equal(a2q_s[loc], ref_s["a2q"][loc]) and \
                torch.equal(a2s_s[loc].view(torch.int32), ref_s["a2s"][loc].view(torch.int32)), f"separate order (bs={bs})"
        # the optional fused-scale order: last-ulp differences in fp32, within the tolerance of the ORACLE
        out_f, a2q_f, a2s_f = run_with_intermediates(layer, weights, x, tw, ids, emap, dev, bs,
                                                     _lib.LO_GEMM_FUSED_SCALE, tokens)
        assert within_tolerance(out_f[tokens].cpu(), ref["out"]), f"fused-scale order out of tolerance (bs={bs})"
        if loc.any():
            frac = (a2q_f[loc] != ref["a2q"][loc]).float().mean().item()
            say(f"  fused-scale order: {100 * frac:.3f} % of the sampled a2q bytes differ from the oracle, "
                f"{100 * (a2s_f[loc] != ref['a2s'][loc]).float().mean().item():.3f} % of the scales")
            assert frac < 0.05
            d = (a2q_f[loc].int() - ref["a2q"][loc].int()).abs()
            assert d.max() <= 2, "a re-quantised activation moved by more than two steps"
        full = out_f.float() - outs[0].float()
        assert full.abs().max() <= 1e-2 * outs[0].float().abs().max()


def test_full_deepseek_v3_zipf_routing(dev, oracle):
    """The full DeepSeek-V3 benchmark configuration at its real width: all 256 experts resident (11.3 GB
    of int8 weights, generated on the device), H=7168, I=2048, Zipf-skewed grouped routing, M=8192, block
    sizes 16..128.  Sampled tokens against the oracle (output rows, a2q, a2s: bit-exact in the
    default order); the block size changes padding and tiling, never the result."""
    from lightop_amd import workloads as wl

    layer = wl.DSV3_FULL
    weights = layer_weights(layer, dev)
    M = 8192
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=5))
    counts = torch.bincount(ids.reshape(-1).long().cpu(), minlength=256)
    assert counts.max() > 4 * counts.float().mean(), "routing is not skewed"
    tokens = torch.tensor([0, 17, 4095, 8191], device=dev)
    ref = oracle_rows(oracle, layer, weights, x, tw, ids, None, tokens, 16, intermediates=True)
    base = None
    for bs in (128, 64, 32, 16):
        say(f"full deepseek-v3 zipf M={M} bs={bs} (max slots/expert {int(counts.max())}, min {int(counts.min())})")
        out, a2q, a2s = run_with_intermediates(layer, weights, x, tw, ids, None, dev, bs, 0, tokens)
        assert torch.equal(out[tokens].cpu().view(torch.int16), ref["out"].view(torch.int16)), f"bs={bs}"
        assert torch.equal(a2q, ref["a2q"]) and torch.equal(a2s.view(torch.int32), ref["a2s"].view(torch.int32)), f"bs={bs}"
        if base is None:
            base = out
        else:
            assert torch.equal(out.view(torch.int16), base.view(torch.int16)), f"bs={bs} changes the result"
    _weights.clear()  # 22 GB of device memory back before the next module
    torch.cuda.empty_cache()


@pytest.mark.parametrize("M,E,k,bs", [(8192, 256, 8, 128), (16384, 256, 8, 16), (4096, 128, 8, 64)])
def test_align_properties_at_full_size(dev, M, E, k, bs):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import moe_align_block_size

    say(f"align properties S={M * k} E={E} bs={bs}")
    layer = wl.MoeLayer("a", E=E, E_global=E, top_k=k, H=128, I=128, routing="softmax")
    ids = wl.make_inputs(layer, M, seed=9)[2].to(dev)
    s, e, p = moe_align_block_size(ids, bs, E)
    torch.cuda.synchronize()
    S = M * k
    flat = ids.reshape(-1).long()
    counts = torch.bincount(flat, minlength=E)
    padded = (counts + bs - 1) // bs * bs
    P = int(p.item())
    assert P == int(padded.sum())
    body = s[:P].long()
    valid = body[body < S]
    assert valid.numel() == S and torch.equal(valid.sort().values, torch.arange(S, device=dev))
    assert (s[P:] == S).all() and (e[P // bs:] == -1).all()
    blocks = body.view(-1, bs)
    owner = e[: P // bs].long()
    assert (owner[1:] >= owner[:-1]).all()
    row_expert = torch.where(blocks < S, flat[blocks.clamp(max=S - 1)], owner[:, None].expand_as(blocks))
    assert (row_expert == owner[:, None]).all()
    # stable: inside an expert the slot ids ascend, pads come last
    assert (blocks.reshape(-1)[1:][(owner.repeat_interleave(bs)[1:] == owner.repeat_interleave(bs)[:-1])]
            >= blocks.reshape(-1)[:-1][(owner.repeat_interleave(bs)[1:] == owner.repeat_interleave(bs)[:-1])]).all()


def test_quant_properties_at_full_size(dev):
    from lightop_amd.quant import per_token_group_quant_int8

    say("quant properties 32768 x 2048")
    g = torch.Generator(device="cuda").manual_seed(1)
    x = (torch.randn(32768, 2048, generator=g, device=dev) * 3).to(torch.bfloat16)
    q, s = per_token_group_quant_int8(x, 128)
    torch.cuda.synchronize()
    xf = x.float().view(-1, 128)
    amax = xf.abs().amax(dim=1).clamp(min=1e-10)
    # IEEE division on the host: a GPU library may turn x / 127 into x * (1 / 127)
    assert torch.equal(s.view(-1).cpu(), amax.cpu() / 127.0)
    qf = q.view(-1, 128).float()
    assert (qf.abs().amax(dim=1) >= 126).all() and qf.abs().max() <= 127
    # truncation toward zero: |q| * s <= |x| and |x| - |q| * s < s (up to one rounding of the division)
    recon = qf.abs() * s.view(-1, 1)
    assert (recon <= xf.abs() * (1 + 2e-7) + 1e-30).all()
    assert (xf.abs() - recon < s.view(-1, 1) * (1 + 1e-6)).all()
    assert (torch.sign(qf) * torch.sign(xf) >= 0).all()
