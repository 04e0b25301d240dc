"""Synthetic block-INT8 MoE workloads: layer shapes, weights, activations and routing.

Weights: int8 uniform in [-127, 127] with one fp32 scale per 128x128 block drawn
lognormal(mu = ln 1e-3, sigma = 0.3).  Activations: bf16 ~ N(0, 1).  Routing: softmax
top-k (renormalised), DeepSeek-V3 grouped sigmoid top-k (8 groups, top-4 groups, group
score = sum of the group's two best experts, renormalised, x2.5; reference form:
test/ci_tests/test_fused_moe_gate.py:9-61), optionally Zipf-skewed.  Everything is
drawn from a seeded torch.Generator on the CPU (or, for layers too large to copy, on
the device) so that a CPU checker and the GPU see the same bits.  Exponentials (the
lognormal scales, softmax, sigmoid) and the renormalising sums are taken in float64 and
rounded to float32 once: torch's float32 exp differs in the last place between CPUs
(vector width), and the committed fixtures must not depend on the host that regenerates
their inputs.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class MoeLayer:
    name: str
    E: int              # experts resident on this GPU
    E_global: int       # experts the router chooses from
    top_k: int
    H: int
    I: int
    routing: str        # "softmax" | "grouped_sigmoid" | "grouped_sigmoid_zipf"
    n_group: int = 1
    topk_group: int = 1
    routed_scaling: float = 1.0
    weight_bits: int = 8  # 8: block-INT8 (128x128 scales); 4: packed int4, one scale per row and 128-wide K group
    quant: str = "block"  # "channel": int8 weights with one scale per row, activations one scale per token

    @property
    def weight_bytes(self) -> int:
        return self.E * 3 * self.I * self.H * self.weight_bits // 8


TINY = MoeLayer("tiny-e8", E=8, E_global=8, top_k=2, H=1024, I=512, routing="softmax")
QWEN3_30B = MoeLayer("qwen3-30b-a3b", E=128, E_global=128, top_k=8, H=2048, I=768, routing="softmax")
DSV3_EP = MoeLayer("deepseek-v3-ep8-share", E=32, E_global=256, top_k=8, H=7168, I=2048,
                   routing="grouped_sigmoid", n_group=8, topk_group=4, routed_scaling=2.5)
DSV3_FULL = MoeLayer("deepseek-v3-full", E=256, E_global=256, top_k=8, H=7168, I=2048,
                     routing="grouped_sigmoid_zipf", n_group=8, topk_group=4, routed_scaling=2.5)

# Qwen3-235B-A22B-shaped layer with int8 weights in the block form: a third shape class for the tile table
# (H = 4096 between the other two layers' 2048 and 7168, I = 1536)
QWEN3_235B = MoeLayer("qwen3-235b-a22b", E=128, E_global=128, top_k=8, H=4096, I=1536, routing="softmax")

TINY_W4 = MoeLayer("tiny-e8-w4a8", E=8, E_global=8, top_k=2, H=1024, I=512, routing="softmax", weight_bits=4)
QWEN3_235B_W4 = MoeLayer("qwen3-235b-a22b-w4a8", E=128, E_global=128, top_k=8, H=4096, I=1536, routing="softmax",
                         weight_bits=4)

# the reference's own int4 form: scales per token and per weight row, both in the epilogue
TINY_W4_PC = MoeLayer("tiny-e8-w4a8-channel", E=8, E_global=8, top_k=2, H=1024, I=512, routing="softmax",
                      weight_bits=4, quant="channel")
QWEN3_235B_W4_PC = MoeLayer("qwen3-235b-a22b-w4a8-channel", E=128, E_global=128, top_k=8, H=4096, I=1536,
                            routing="softmax", weight_bits=4, quant="channel")

TINY_PC = MoeLayer("tiny-e8-channel", E=8, E_global=8, top_k=2, H=1024, I=512, routing="softmax", quant="channel")
QWEN3_30B_PC = MoeLayer("qwen3-30b-a3b-channel", E=128, E_global=128, top_k=8, H=2048, I=768, routing="softmax",
                        quant="channel")
DSV3_EP_PC = MoeLayer("deepseek-v3-ep8-share-channel", E=32, E_global=256, top_k=8, H=7168, I=2048,
                      routing="grouped_sigmoid", n_group=8, topk_group=4, routed_scaling=2.5, quant="channel")

LAYERS = {l.name: l for l in (TINY, QWEN3_30B, DSV3_EP, DSV3_FULL, QWEN3_235B, TINY_W4, QWEN3_235B_W4, TINY_W4_PC,
                              QWEN3_235B_W4_PC, TINY_PC, QWEN3_30B_PC, DSV3_EP_PC)}


def make_weights(layer: MoeLayer, seed: int = 0, device="cpu", gen_device: Optional[str] = None):
    """(w1 [E,2I,H] int8, w2 [E,H,I] int8, w1_scale [E,2I/128,H/128], w2_scale [E,H/128,I/128]); for a
    per-channel layer the scales are [E,2I,1] and [E,H,1]; for a
    4-bit layer (w1 [E,2I,H/2], w2 [E,H,I/2] uint8: int4 uniform in [-8, 7], two per byte along K, even k
    in the high nibble; w1_scale [E,2I,H/128], w2_scale [E,H,I/128], or [E,2I,1] and [E,H,1] in the
    per-channel form, whose sums carry the factor 16 of the nibbles)."""
    gen_device = gen_device or "cpu"
    g = torch.Generator(device=gen_device).manual_seed(seed)
    E, H, I = layer.E, layer.H, layer.I
    if layer.weight_bits == 4:
        def w4(shape):  # packed bytes: both nibbles uniform, i.e. both elements uniform in [-8, 7]
            return torch.randint(0, 256, shape, generator=g, dtype=torch.int16, device=gen_device).to(torch.uint8)

        def s4(shape):
            z = torch.randn(shape, generator=g, dtype=torch.float32, device=gen_device) * 0.3 + math.log(1e-2)
            return torch.exp(z.double()).float()

        if layer.quant == "channel":
            return tuple(t.to(device) for t in (w4((E, 2 * I, H // 2)), w4((E, H, I // 2)),
                                                s4((E, 2 * I, 1)) / 16, s4((E, H, 1)) / 16))
        return tuple(t.to(device) for t in (w4((E, 2 * I, H // 2)), w4((E, H, I // 2)),
                                            s4((E, 2 * I, H // 128)), s4((E, H, I // 128))))

    def w(shape):
        return torch.randint(-127, 128, shape, generator=g, dtype=torch.int8, device=gen_device)

    def s(shape):
        z = torch.randn(shape, generator=g, dtype=torch.float32, device=gen_device) * 0.3 + math.log(1e-3)
        return torch.exp(z.double()).float()

    w1 = w((E, 2 * I, H))
    w2 = w((E, H, I))
    if layer.quant == "channel":  # one scale per weight row (the reference's shape, [E, N, 1])
        return tuple(t.to(device) for t in (w1, w2, s((E, 2 * I, 1)), s((E, H, 1))))
    w1s = s((E, 2 * I // 128, H // 128))
    w2s = s((E, H // 128, I // 128))
    return tuple(t.to(device) for t in (w1, w2, w1s, w2s))


def expert_map_for(layer: MoeLayer, device="cpu") -> Optional[torch.Tensor]:
    """Global id -> local id for the first ``E`` experts, -1 elsewhere; None if all are local."""
    if layer.E == layer.E_global:
        return None
    m = torch.full((layer.E_global,), -1, dtype=torch.int32)
    m[: layer.E] = torch.arange(layer.E, dtype=torch.int32)
    return m.to(device)


def route(layer: MoeLayer, logits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(topk_weights [M,k] f32, topk_ids [M,k] int32) from router logits [M, E_global]."""
    k = layer.top_k
    if layer.routing == "softmax":
        p = torch.softmax(logits.double(), dim=-1)
        w, ids = torch.topk(p, k, dim=-1)
        w = w / w.sum(dim=-1, keepdim=True)
        return w.float().contiguous(), ids.to(torch.int32).contiguous()
    scores = torch.sigmoid(logits.double())
    M, Eg = scores.shape
    per = Eg // layer.n_group
    group_scores = scores.view(M, layer.n_group, per).topk(2, dim=-1)[0].sum(dim=-1)
    gidx = torch.topk(group_scores, layer.topk_group, dim=-1, sorted=False)[1]
    gmask = torch.zeros_like(group_scores)
    gmask.scatter_(1, gidx, 1.0)
    mask = gmask.unsqueeze(-1).expand(M, layer.n_group, per).reshape(M, Eg)
    masked = scores.masked_fill(mask == 0, float("-inf"))
    ids = torch.topk(masked, k, dim=-1, sorted=False)[1]
    w = scores.gather(1, ids)
    w = w / w.sum(dim=-1, keepdim=True) * layer.routed_scaling
    return w.float().contiguous(), ids.to(torch.int32).contiguous()


def make_inputs(layer: MoeLayer, M: int, seed: int = 0, device="cpu"):
    """(x [M,H] bf16, topk_weights [M,k] f32, topk_ids [M,k] int32) for one step."""
    g = torch.Generator(device="cpu").manual_seed(seed * 7919 + M)
    x = torch.randn((M, layer.H), generator=g, dtype=torch.float32).to(torch.bfloat16)
    logits = torch.randn((M, layer.E_global), generator=g, dtype=torch.float32)
    if layer.routing.endswith("zipf"):
        perm = torch.randperm(layer.E_global, generator=g)
        zipf = 1.0 / torch.arange(1, layer.E_global + 1, dtype=torch.float64) ** 1.2
        bias = torch.empty(layer.E_global)
        bias[perm] = torch.log(zipf / zipf.sum()).float()
        logits = logits + bias
    w, ids = route(layer, logits)
    return x.to(device), w.to(device), ids.to(device)


def algorithmic_work(layer: MoeLayer, topk_ids: torch.Tensor, expert_map: Optional[torch.Tensor]):
    """(int8 ops, bytes, local slots, active local experts) of one call: ops = 6*S_loc*I*H;
    bytes = every active expert's weights and block scales once + bf16 activations in and
    out + routing tensors.  Intermediates are not counted."""
    ids = topk_ids.reshape(-1).long().cpu()
    local = ids if expert_map is None else expert_map.cpu().long()[ids]
    local = local[local >= 0]
    S_loc = int(local.numel())
    E_act = int(torch.unique(local).numel())
    H, I = layer.H, layer.I
    M = topk_ids.shape[0]
    if layer.weight_bits == 4 and layer.quant == "channel":  # half a byte per weight, one scale per row
        per_expert = 3 * I * H // 2 + 4 * (2 * I + H)
    elif layer.weight_bits == 4:  # half a byte per weight, one scale per row and K group
        per_expert = 3 * I * H // 2 + 4 * (2 * I * (H // 128) + H * (I // 128))
    elif layer.quant == "channel":
        per_expert = 3 * I * H + 4 * (2 * I + H)
    else:
        per_expert = 3 * I * H + 4 * ((2 * I // 128) * (H // 128) + (H // 128) * (I // 128))
    nbytes = E_act * per_expert + 2 * M * H * 2 + M * layer.top_k * 8
    return 6 * S_loc * I * H, nbytes, S_loc, E_act
