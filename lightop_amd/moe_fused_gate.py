"""Grouped top-k router (reference: python/lightop/moe_fused_gate.py:10-31)."""
from . import op


def moe_fused_gate(
    x,
    bias,
    num_expert_group,
    topk_group,
    topk,
    n_share_experts_fusion,
    routed_scaling_factor,
    apply_routed_scaling_factor_on_output=True,
    output_indices_int64=False,
):
    return op.moe_fused_gate(
        x,
        bias,
        num_expert_group,
        topk_group,
        topk,
        n_share_experts_fusion,
        routed_scaling_factor,
        apply_routed_scaling_factor_on_output,
        output_indices_int64,
    )
