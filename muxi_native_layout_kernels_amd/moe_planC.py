"""Fused MoE layer entry point; same signature and defaults as the reference's
`muxi_moe_planC.fused_moe` (muxi_layout_kernels/muxi_moe_planC.py:6-149).

One library call per layer (`mlk_fused_moe`): router (scores, grouped selection,
top-K and the optional renormalisation), alignment, grouped gate/up GeMM and
grouped down GeMM.  Apart from the output
nothing is allocated after the first call of a given shape: routing tables and
the kernel workspace are cached per device and stream and are never freed, so a
HIP graph captured around this function stays valid whatever runs later.
"""
import threading
from typing import List, Optional

import torch

from . import ops

_cache_lock = threading.Lock()
_route_cache = {}
_plans = {}


def _routing_buffers(n_tokens, topk, dtype, device, stream=None):
    """Routing tables (ids, weights) per shape, device and stream.  Entries are never dropped: the kernels get
    raw pointers, and a HIP graph captured by the caller keeps using them.  An entry is a few bytes per token."""
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    key = (n_tokens, topk, dtype, device.type, device.index, int(stream))
    with _cache_lock:
        hit = _route_cache.get(key)
        if hit is None:
            hit = (torch.empty(n_tokens, topk, dtype=torch.int32, device=device),
                   torch.empty(n_tokens, topk, dtype=dtype, device=device))
            _route_cache[key] = hit
        return hit


def fused_moe(
    hidden_states: torch.Tensor,  # [batch_size, hidden_size]
    w1: torch.Tensor,             # [E, 2I, H] per-expert layout-A slabs (or [E, 2I/16, H/8, 16, 8])
    w2: torch.Tensor,             # [E, H, I]
    gating_output: torch.Tensor,  # [batch_size, num_experts]
    topk: int,
    renormalize: bool,
    use_grouped_topk: bool = False,
    num_expert_group: Optional[int] = None,
    topk_group: Optional[int] = None,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    gating_bias: Optional[torch.Tensor] = None,
    score_func: str = "softmax",
    soft_fp8: bool = False,
    APerWarp: int = 2,
    splitK: int = 3,
    tile_m_2: int = 128,
    tile_n_2: int = 16,
    tile_k_2: int = 128,
    block_dim_x_gemm: int = 256,
    experts_map: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The MetaX tile parameters (APerWarp .. block_dim_x_gemm) are accepted and ignored."""
    # A combination of shapes, dtypes, devices and options that has passed every check below before runs from its
    # launch plan: per call only contiguity is checked again (a shape does not tell it).
    key = (hidden_states.shape, hidden_states.dtype, hidden_states.device, w1.shape, w1.dtype, w1.device, w2.shape,
           w2.dtype, w2.device, gating_output.shape, gating_output.dtype, gating_output.device, topk, bool(renormalize),
           use_grouped_topk, num_expert_group, topk_group, score_func, soft_fp8,
           None if w1_scale is None else (w1_scale.shape, w1_scale.dtype, w1_scale.device),
           None if w2_scale is None else (w2_scale.shape, w2_scale.dtype, w2_scale.device),
           None if block_shape is None else tuple(block_shape),
           None if gating_bias is None else (gating_bias.shape, gating_bias.dtype, gating_bias.device),
           None if experts_map is None else (experts_map.shape, experts_map.dtype, experts_map.device))
    plan = _plans.get(key)
    if plan is not None and hidden_states.is_contiguous() and w1.is_contiguous() and w2.is_contiguous() and \
            gating_output.is_contiguous() and (w1_scale is None or w1_scale.is_contiguous()) and \
            (w2_scale is None or w2_scale.is_contiguous()) and (gating_bias is None or gating_bias.is_contiguous()) and \
            (experts_map is None or experts_map.is_contiguous()):
        B, H, E, I, w_kind, score_fun, n_groups, k_groups, scaled = plan
        topk_ids, topk_weights = _routing_buffers(B, topk, hidden_states.dtype, hidden_states.device,
                                                  ops._stream_of(hidden_states))
        y = torch.empty_like(hidden_states)
        ops.fused_moe_raw(w1, w2, hidden_states, gating_output, B, E, topk, H, I, w_kind, score_fun, n_groups, k_groups,
                          gating_bias, renormalize, experts_map, w1_scale if scaled else None,
                          w2_scale if scaled else None, topk_ids, topk_weights, y)
        return y
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    if num_expert_group is None:
        num_expert_group = 1
    if topk_group is None:
        topk_group = 1
    if not use_grouped_topk and num_expert_group != 1:
        raise ValueError("When use_grouped_topk is False, num_expert_group must be 1.")
    if score_func == "softmax":
        score_fun = 0
    elif score_func == "sigmoid":
        score_fun = 1
    else:
        raise ValueError("Unsupported scoring function")

    shape = hidden_states.size()
    B, H = hidden_states.shape
    ops._check(hidden_states.is_cuda and hidden_states.is_contiguous(), "hidden_states must be a contiguous CUDA tensor")
    ops._check(hidden_states.dtype in ops._KIND, "hidden_states must be fp16 or bf16")
    ops._check(gating_output.dtype == hidden_states.dtype, "gating_output must have the activation dtype")
    # the router's argument checks (ops.fused_routing_gate), done here because one library call runs the whole layer
    n_router_experts = gating_output.size(-1)
    ops._check(gating_output.is_cuda and gating_output.is_contiguous(), "gating_output must be a contiguous CUDA tensor")
    ops._check(B * n_router_experts == gating_output.numel(), "batch_size does not match gating_output")
    ops._check(1 <= n_router_experts <= 256, "the router supports at most 256 experts")
    ops._check(num_expert_group >= 1 and n_router_experts % num_expert_group == 0,
               "n_groups must divide the number of experts")
    ops._check(1 <= topk_group <= num_expert_group, "topK_groups must be in 1..n_groups")
    ops._check(1 <= topk <= min(32, n_router_experts), "topK must be in 1..min(32, experts)")
    if gating_bias is not None:
        ops._check(gating_bias.dtype == gating_output.dtype, "Mismatched dtypes: load_balance_bias and gating_output.")
    topk_ids, topk_weights = _routing_buffers(B, topk, hidden_states.dtype, hidden_states.device)

    if w1.dim() == 5:
        e1, m1, k1 = w1.shape[0], w1.shape[1] * 16, w1.shape[2] * 8
        e2, m2, k2 = w2.shape[0], w2.shape[1] * 16, w2.shape[2] * 8
    else:
        e1, m1, k1 = w1.shape
        e2, m2, k2 = w2.shape
    assert e1 == e2
    assert k1 == m2
    ops._check(k1 == H and m1 == 2 * k2, "w1 must be [E, 2I, H] and w2 [E, H, I]")
    ops._check(w1.is_cuda and w2.is_cuda and w1.is_contiguous() and w2.is_contiguous(),
               "expert weights must be contiguous CUDA tensors")
    ops._check(H % 128 == 0 and k2 % 128 == 0, "hidden and intermediate sizes must be multiples of 128")

    if soft_fp8:
        assert w1_scale is not None and w2_scale is not None
        ops._check(w1.element_size() == 1 and w2.element_size() == 1, "soft_fp8 needs one e4m3 byte per weight")
        ops._check(hidden_states.dtype == torch.bfloat16, "Weight date type and activation date type mismatch")
        ops._check(block_shape is not None and list(block_shape) == [128, 128],
                   "block_shape must be (128, 128) for float8_e4m3fn.")
        ops._check(w1_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32, "scales must be float32.")
        ops._check(tuple(w1_scale.shape) == (e1, m1 // 128, k1 // 128) and w1_scale.is_contiguous(),
                   "w1_scale must be [E, 2I/128, H/128]")
        ops._check(tuple(w2_scale.shape) == (e2, m2 // 128, k2 // 128) and w2_scale.is_contiguous(),
                   "w2_scale must be [E, H/128, I/128]")
        w_kind = ops._FP8_KIND
    else:
        ops._check(w1.dtype == hidden_states.dtype and w2.dtype == hidden_states.dtype,
                   "Weight date type and activation date type mismatch")
        w_kind = ops._KIND[w1.dtype]
        w1_scale = w2_scale = None
    if experts_map is not None and experts_map.dtype != torch.int:
        experts_map = experts_map.to(torch.int)

    y = torch.empty_like(hidden_states)
    ops.fused_moe_raw(w1, w2, hidden_states, gating_output, B, e1, topk, H, k2, w_kind, score_fun, num_expert_group,
                      topk_group, gating_bias, renormalize, experts_map, w1_scale, w2_scale, topk_ids, topk_weights, y)
    if experts_map is None or experts_map.dtype == torch.int:      # (a converted map is a new tensor every call)
        _plans[key] = (B, H, e1, k2, w_kind, score_fun, num_expert_group, topk_group, w1_scale is not None)
    return y.view(shape)
