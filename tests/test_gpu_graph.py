"""The whole path recorded into a HIP graph: every replay must reproduce the eager result.

The entry points allocate nothing and never synchronise, so a caller may capture them.
The replays are separated by eager work and synchronisations of the program itself."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M", [1, 16, 64])
@pytest.mark.parametrize("form", ["block", "block_preshuffled", "channel", "w4"])
def test_graph_replays_match_eager(M, form):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import (fused_experts_impl_int8, fused_experts_impl_w4a8, preshuffle_moe_scale_int4,
                                 preshuffle_moe_weight, preshuffle_moe_weight_int4)

    _lib.lib()
    dev = torch.device("cuda:0")
    layer = {"block": wl.TINY, "block_preshuffled": wl.TINY, "channel": wl.TINY_PC, "w4": wl.TINY_W4}[form]
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev)
    if form == "w4":
        w1, w2 = preshuffle_moe_weight_int4(w1), preshuffle_moe_weight_int4(w2)
        w1s, w2s = preshuffle_moe_scale_int4(w1s), preshuffle_moe_scale_int4(w2s)
    if form == "block_preshuffled":  # load-time layout: the two-launch path at 1 and 16 tokens
        w1, w2 = preshuffle_moe_weight(w1), preshuffle_moe_weight(w2)
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=5))
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)

    def run():
        if form == "w4":
            return fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13, w1_scale=w1s, w2_scale=w2s,
                                           block_shape=[1, 128])
        return fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True,
                                       per_channel_quant=form == "channel", w1_scale=w1s, w2_scale=w2s,
                                       block_shape=None if form == "channel" else [128, 128])

    print(f"[case] graph replay M={M} {form}", flush=True)
    eager = run().clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = run()
    for rep in range(4):
        out.zero_()
        cache13.fill_(float(rep))                 # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {rep} differs"
