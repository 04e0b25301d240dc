"""The whole-path entry point that allocates nothing (lo_fused_experts_block_int8_noalloc): its
output must equal that of lo_fused_experts_block_int8 with a caller workspace, bit for bit, on two
calls in a row that share the library's built-in scratch, the second on a smaller input; problems
beyond the built-in scratch are refused.  Everything goes through the C ABI with ctypes."""
import ctypes
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


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def call_both(dev, layer, M, seed, weights, bs, flags):
    """(out of the workspace form, out of the no-alloc form) for one batch."""
    from lightop_amd import _lib, workloads as wl

    lib = _lib.lib()
    w1, w2, w1s, w2s = weights
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=seed))
    emap = wl.expert_map_for(layer, dev)
    k, H, I = layer.top_k, layer.H, layer.I
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    outs = []
    for noalloc in (False, True):
        cache3 = torch.full((M * k * H,), float("nan"), dtype=torch.bfloat16, device=dev)
        out = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
        head = (_p(x), _lib.LO_BF16, M, H, I, layer.E, layer.E_global, k, _p(w1), _p(w1s), _p(w2), _p(w2s), _p(tw),
                _p(ids), _lib.LO_I32, _p(emap), 0, ctypes.c_float(layer.routed_scaling), _p(None), _p(cache3), _p(out))
        if noalloc:
            rc = lib.lo_fused_experts_block_int8_noalloc(*head, bs, flags, stream)
        else:
            n = lib.lo_fused_experts_workspace_bytes(M, k, H, I, layer.E_global, 0)
            ws = torch.empty(n + 256, dtype=torch.uint8, device=dev)
            wp = (ws.data_ptr() + 255) // 256 * 256
            rc = lib.lo_fused_experts_block_int8(*head, ctypes.c_void_p(wp), n, bs, flags, stream)
        _lib.check(rc)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    return outs


@pytest.mark.parametrize("name,sizes", [("tiny-e8", (200, 7)), ("deepseek-v3-ep8-share", (96, 5)),
                                        ("qwen3-30b-a3b", (1024, 33))])
def test_noalloc_entry_point_matches_the_workspace_form(dev, name, sizes):
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.LAYERS[name]
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
    weights = (preshuffle_moe_weight(w1), preshuffle_moe_weight(w2), w1s, w2s)
    del w1, w2
    for call, M in enumerate(sizes):  # two calls in a row on the shared scratch, the second one smaller
        for bs in (0, 16):
            say(f"noalloc {name} call {call} M={M} bs={bs}")
            a, b = call_both(dev, layer, M, 11 + call, weights, bs, _lib.LO_GEMM_W_PRESHUFFLED)
            assert not torch.isnan(a.float()).any() and not torch.isnan(b.float()).any()
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"M={M} bs={bs}"


def test_noalloc_entry_point_refuses_what_does_not_fit(dev):
    from lightop_amd import _lib

    lib = _lib.lib()
    M, k, H, I, E = 8192, 8, 2048, 768, 128
    assert lib.lo_fused_experts_workspace_bytes(M, k, H, I, E, 128) > _lib.LO_NOALLOC_SCRATCH_BYTES
    buf = torch.zeros(1024, dtype=torch.uint8, device=dev)  # never touched: the size check comes first
    p = _p(buf)
    rc = lib.lo_fused_experts_block_int8_noalloc(p, _lib.LO_BF16, M, H, I, E, E, k, p, p, p, p, p, p, _lib.LO_I32,
                                                 _p(None), 0, ctypes.c_float(1.0), _p(None), p, p, 128, 0,
                                                 ctypes.c_void_p(0))
    assert rc == -2 and b"built-in scratch holds" in lib.lo_last_error()
