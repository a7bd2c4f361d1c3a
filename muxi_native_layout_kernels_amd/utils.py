"""Torch helpers that ship beside the kernels, mirroring the reference's
`muxi_layout_kernels/utils.py`: the block-scale helpers used to build soft-FP8
expected weights (:7-25) and a pure-torch MoE on un-packed weights (:131-244)
that callers use as a slow cross-check on any device.  Nothing here calls the
HIP library except the two thin wrappers kept for name compatibility.
"""
from typing import Optional

import torch
import torch.nn.functional as F

from . import ops


def scale_tensor(weight, scale):
    """Multiply every 128x128 block of `weight` [m, k] by its entry of `scale`
    [ceil(m/128), ceil(k/128)], in the weight's dtype (reference utils.py:14-25)."""
    m, k = weight.shape
    factors = scale.to(weight.dtype).repeat_interleave(128, dim=0)[:m].repeat_interleave(128, dim=1)[:, :k]
    return weight * factors


def scale_whole_tensor(weight, scale):
    """Per-expert `scale_tensor` on a bf16 copy of `weight` [e, m, k] (reference utils.py:7-12)."""
    out = weight.clone().to(torch.bfloat16)
    for expert in range(out.shape[0]):
        out[expert] = scale_tensor(out[expert], scale[expert])
    return out


def routing_gate(*args, **kwargs):
    return ops.routing_gate(*args, **kwargs)


def experts_compute(*args, **kwargs):
    return ops.experts_compute(*args, **kwargs)


def _select_experts(gating_output, topk, num_expert_group, topk_group, renormalize, bias, score_func, dtype):
    if score_func == "softmax":
        scores = torch.softmax(gating_output, dim=-1, dtype=dtype)
    elif score_func == "sigmoid":
        scores = torch.sigmoid(gating_output)
    else:
        raise ValueError("Unsupported scoring function")
    plain = scores
    if bias is not None:
        scores = scores + bias.unsqueeze(0)
    tokens, experts = scores.shape
    groups = max(int(num_expert_group), 1)
    per_group = scores.view(tokens, groups, experts // groups)
    group_score = per_group.topk(2, dim=-1)[0].sum(dim=-1) if bias is not None else per_group.max(dim=-1).values
    kept = torch.topk(group_score, k=topk_group, dim=-1, sorted=False)[1]
    group_mask = torch.zeros_like(group_score).scatter_(1, kept, 1).bool()
    expert_mask = group_mask.unsqueeze(-1).expand(tokens, groups, experts // groups).reshape(tokens, experts)
    masked = scores.masked_fill(~expert_mask, 0.0)
    if bias is not None:
        ids = torch.topk(masked, k=topk, dim=-1, sorted=False)[1]
        weights = plain.gather(1, ids)
    else:
        weights, ids = torch.topk(masked, k=topk, dim=-1, sorted=False)
    if renormalize:
        weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights.to(dtype), ids


def fused_moe(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, gating_output: torch.Tensor,
              topk: int, num_expert_group: int = 0, topk_group: int = 1, global_num_experts: int = 1,
              expert_map: torch.Tensor = None, renormalize: bool = False,
              e_score_correction_bias: Optional[torch.Tensor] = None, score_func: str = "softmax") -> torch.Tensor:
    """Pure-torch MoE on un-packed weights: w1 [E, 2I, H] (gate rows then up rows), w2 [E, H, I].
    Every expert is evaluated on every token and weighted by its (possibly zero) routing weight."""
    orig_shape = hidden_states.shape
    hidden = hidden_states.shape[-1]
    dtype = hidden_states.dtype
    x = hidden_states.reshape(-1, hidden)
    logits = gating_output.reshape(x.shape[0], -1)
    inter = w2.shape[-1]
    weights, ids = _select_experts(logits, topk, num_expert_group, topk_group, renormalize, e_score_correction_bias,
                                   score_func, dtype)
    if expert_map is not None:
        ids = expert_map[ids]
    total = torch.zeros_like(x)
    for expert in range(w1.shape[0]):
        gate_up = F.linear(x, w1[expert])
        act = gate_up[:, inter:] * F.silu(gate_up[:, :inter])
        share = (weights * (ids == expert)).sum(dim=-1, keepdim=True)
        total = total + F.linear(act, w2[expert]) * share
    return total.view(orig_shape)


__all__ = ["scale_tensor", "scale_whole_tensor", "routing_gate", "experts_compute", "fused_moe"]
