"""Whole path on randomly drawn configurations, through the C ABI, bit for bit against the oracle: the four
weight forms, both activations, bf16, fp16 and fp32 rows (fp32: the block form only, refused elsewhere), every block size (a size the form does not offer must be
refused with an error, not computed), row-major and load-time weight layouts, expert maps (leading and
scattered), in-place output, the router weight on the input, shared output with a scaling factor, skewed
routing that fills 128- and 160-token blocks, zero rows."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

FORMS = ("block", "block", "channel", "w4", "w4pc")


def _draw(rnd):
    form = rnd.choice(FORMS)
    E = rnd.choice([1, 2, 3, 4, 6, 8, 12])
    Eg = E * rnd.choice([1, 1, 2, 4])
    top_k = min(rnd.choice([1, 2, 4, 6, 8]), Eg)
    H = 128 * rnd.choice([1, 2, 3, 4, 6, 8, 12, 16])
    I = 128 * rnd.choice([1, 2, 3, 4, 6])
    M = rnd.choice([1, 2, 3, 5, 8, 17, 33, 40, 64, 77, 130, 200, 300, 520, 1000, 2100])
    while M * top_k * 3 * H * I > 3e10:
        M = max(1, M // 2)
    return dict(form=form, E=E, Eg=Eg, top_k=top_k, H=H, I=I, M=M,
                dtype=rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32]),
                act=rnd.choice(["silu", "silu", "gelu"]), bs=rnd.choice([0, 0, 16, 32, 64, 128, 160]),
                pre=rnd.random() < 0.8 or form in ("w4", "w4pc"), inplace=rnd.random() < 0.2,
                on_input=rnd.random() < 0.2, with_shared=rnd.random() < 0.3, rsf=rnd.choice([1.0, 1.0, 2.5, 0.5]),
                skew=rnd.random() < 0.4, x_scale=rnd.choice([0.3, 1.0, 3.0]), zero_row=rnd.random() < 0.3,
                renorm=rnd.random() < 0.5, scattered_map=rnd.random() < 0.5)


def _block_size_offered(c):
    """160-token blocks: weights in the load-time layout with block scales (2I <= H) or per-channel scales."""
    if c["bs"] != 160:
        return True
    if c["form"] == "w4pc" or (c["form"] == "channel" and c["pre"]):
        return True
    return c["form"] == "block" and c["pre"] and 2 * c["I"] <= c["H"] and c["dtype"] != torch.float32


@pytest.mark.parametrize("seed", [11, 12])
def test_random_configurations_bit_exact(oracle, seed):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import workloads as wl
    from lightop_amd.moe import (fused_experts_impl_int8, fused_experts_impl_w4a8, preshuffle_moe_weight,
                                 preshuffle_moe_weight_int4)

    dev = torch.device("cuda:0")
    refused = 0
    for case in range(150):
        rnd = random.Random(seed * 100003 + case)
        c = _draw(rnd)
        print(f"[case] random {seed}:{case} " + " ".join(f"{k}={v}" for k, v in c.items()), flush=True)
        E, Eg, k, H, I, M, dtype = c["E"], c["Eg"], c["top_k"], c["H"], c["I"], c["M"], c["dtype"]
        layer = wl.MoeLayer("random", E=E, E_global=Eg, top_k=k, H=H, I=I, routing="softmax",
                            weight_bits=4 if c["form"] in ("w4", "w4pc") else 8,
                            quant="channel" if c["form"] in ("channel", "w4pc") else "block")
        g = torch.Generator().manual_seed(seed * 7 + case)
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=case)
        x = (torch.randn(M, H, generator=g) * c["x_scale"]).to(dtype)
        if c["zero_row"] and M > 2:
            x[rnd.randrange(M)] = 0
        logits = torch.randn(M, Eg, generator=g)
        if c["skew"]:
            logits[:, 0] += 4.0
        tw, ids = torch.topk(torch.softmax(logits, -1), k, dim=-1)
        if c["renorm"]:
            tw = tw / tw.sum(-1, keepdim=True)
        ids, tw = ids.to(torch.int32).contiguous(), tw.contiguous()
        emap = wl.expert_map_for(layer)
        if emap is not None and c["scattered_map"]:
            held = torch.randperm(Eg, generator=g)[:E]
            emap = torch.full((Eg,), -1, dtype=torch.int32)
            emap[held] = torch.arange(E, dtype=torch.int32)
        shared = (torch.randn(M, H, generator=g) * 0.1).to(dtype) if c["with_shared"] else None
        if layer.weight_bits == 4:
            wd1, wd2 = preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev))
        elif c["pre"]:
            wd1, wd2 = preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev))
        else:
            wd1, wd2 = w1.to(dev), w2.to(dev)
        cache13 = torch.empty(M * k * max(2 * I, H), dtype=dtype, device=dev)
        common = dict(global_num_experts=Eg, expert_map=None if emap is None else emap.to(dev),
                      w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), activation=c["act"],
                      lightop_amd_block_size_m=c["bs"], inplace=c["inplace"],
                      apply_router_weight_on_input=c["on_input"], routed_scaling_factor=c["rsf"],
                      shared_output=None if shared is None else shared.to(dev))

        def run():
            if c["form"] in ("w4", "w4pc"):
                return fused_experts_impl_w4a8(x.to(dev), wd1, wd2, tw.to(dev), ids.to(dev), cache13,
                                               block_shape=None if c["form"] == "w4pc" else [1, 128], **common)
            if c["form"] == "channel":
                return fused_experts_impl_int8(x.to(dev), wd1, wd2, tw.to(dev), ids.to(dev), cache13,
                                               use_int8_w8a8=True, per_channel_quant=True, block_shape=None, **common)
            return fused_experts_impl_int8(x.to(dev), wd1, wd2, tw.to(dev), ids.to(dev), cache13, use_int8_w8a8=True,
                                           block_shape=[128, 128], **common)

        if dtype == torch.float32 and c["form"] != "block":  # fp32 rows: the block form with int8 weights only
            with pytest.raises(NotImplementedError):
                run()
            refused += 1
            continue
        if not _block_size_offered(c):
            with pytest.raises(RuntimeError, match="block_size_m 160"):
                run()
            refused += 1
            continue
        out = run()
        torch.cuda.synchronize()
        fn = {"block": oracle.fused_experts_block_int8, "channel": oracle.fused_experts_channel_int8,
              "w4": oracle.fused_experts_w4a8, "w4pc": oracle.fused_experts_w4a8_channel}[c["form"]]
        ref = fn(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=Eg, expert_map=emap,
                 apply_router_weight_on_input=c["on_input"], routed_scaling_factor=c["rsf"], shared_output=shared,
                 activation=c["act"])
        got = out.cpu()
        assert got.dtype == dtype
        nan = ref.isnan()
        assert torch.equal(got.isnan(), nan)
        word = torch.int32 if dtype == torch.float32 else torch.int16
        assert torch.equal(got.view(word)[~nan], ref.view(word)[~nan])
    assert refused < 60  # most draws compute
