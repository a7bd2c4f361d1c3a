"""Fused MoE layer, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Two statements:

* `torch_path_fused_moe` restates the reference's pure-torch MoE
  (muxi_layout_kernels/utils.py:131-244): scores in the activation dtype,
  correction bias for selection only, group mask, library top-k, optional
  renormalisation, then a DENSE loop over all experts with masked routing
  weights.  This is the reference's CPU-runnable path and the one the
  benchmark times on the host cores.
* `moe_expected` is the sparse statement in float64 on un-packed weights from
  given (ids, weights): y_t = sum_k w_tk * W2[e_tk] (silu(G x_t) * (U x_t)),
  with the intermediate rounded to T once, as the HIP path stores it.

Pinned by: the algebraic identity "dense masked sum over experts == gather of
the selected experts" (the two statements must agree when fed the same
routing), and float64 brute force with explicit Python loops on a tiny shape.
"""
import numpy as np
import torch
import torch.nn.functional as F

from . import softfp8


def torch_path_fused_moe(hidden, w1, w2, gating, topk, num_expert_group=1, topk_group=1,
                         renormalize=False, bias=None, score_func="softmax", expert_map=None):
    """Restatement of muxi_layout_kernels/utils.py:131-244 (un-packed w1 [E,2I,H],
    w2 [E,H,I]); runs on whatever device the tensors live on."""
    dtype = hidden.dtype
    n_tok, _ = hidden.shape
    n_exp = w1.shape[0]
    inter = w2.shape[-1]
    if score_func == "softmax":
        sc = torch.softmax(gating, dim=-1, dtype=dtype)          # utils.py:164
    elif score_func == "sigmoid":
        sc = torch.sigmoid(gating)                                 # utils.py:166
    else:
        raise ValueError("Unsupported scoring function")
    plain = sc
    if bias is not None:
        sc = sc + bias.unsqueeze(0)                                # utils.py:167-171
    grouped = sc.view(n_tok, num_expert_group, -1)
    if bias is not None:
        gsc = grouped.topk(2, dim=-1)[0].sum(dim=-1)               # utils.py:176-178
    else:
        gsc = grouped.max(dim=-1).values                           # utils.py:180-181
    gidx = torch.topk(gsc, k=topk_group, dim=-1, sorted=False)[1]  # utils.py:185-186
    gmask = torch.zeros_like(gsc).scatter_(1, gidx, 1)
    emask = gmask.unsqueeze(-1).expand(n_tok, num_expert_group, sc.shape[-1] // num_expert_group)  # utils.py:189-191
    masked = sc.masked_fill(~emask.reshape(n_tok, -1).bool(), 0.0)  # utils.py:192-196
    if bias is not None:
        ids = torch.topk(masked, k=topk, dim=-1, sorted=False)[1]  # utils.py:199
        wts = plain.gather(1, ids)
    else:
        wts, ids = torch.topk(masked, k=topk, dim=-1, sorted=False)  # utils.py:207-210
    if renormalize:
        wts = wts / wts.sum(dim=-1, keepdim=True)                  # utils.py:214-215
    wts = wts.to(dtype)
    if expert_map is not None:
        ids = expert_map[ids]
    out = None
    for e in range(n_exp):                                         # utils.py:229-242
        gate_w = (wts * (ids == e)).sum(dim=-1, keepdim=True)
        proj = F.linear(hidden, w1[e])
        act = proj[:, inter:] * F.silu(proj[:, :inter])
        cur = F.linear(act, w2[e]) * gate_w
        out = cur if out is None else out + cur
    return out


def _f64(t):
    if isinstance(t, torch.Tensor):
        return t.detach().cpu().to(torch.float64).numpy()
    return np.asarray(t, dtype=np.float64)


def moe_expected(hidden, w1, w2, ids, wts, round_h_to=None, expert_map=None):
    """Sparse float64 MoE from given routing.  w1 [E,2I,H], w2 [E,H,I] un-packed
    (any float dtype or float32 ndarray).  ids [T,K] int, wts [T,K].  If
    `round_h_to` is a torch dtype the SiLU*up intermediate is rounded to it
    (through fp32) before the down projection.  Pairs whose mapped expert is -1
    contribute nothing (moe_align_tokens.cu:14-17)."""
    x = _f64(hidden)
    n_tok, hdim = x.shape
    ids_np = np.asarray(ids.cpu() if isinstance(ids, torch.Tensor) else ids).astype(np.int64)
    w_np = _f64(wts)
    inter = w2.shape[-1]
    y = np.zeros((n_tok, hdim), dtype=np.float64)
    cache = {}
    for t in range(n_tok):
        for k in range(ids_np.shape[1]):
            e = int(ids_np[t, k])
            if expert_map is not None:
                e = int(expert_map[e])
                if e == -1:
                    continue
            if e not in cache:
                cache[e] = (_f64(w1[e]), _f64(w2[e]))
            a1, a2 = cache[e]
            proj = a1 @ x[t]
            g, u = proj[:inter], proj[inter:]
            with np.errstate(over="ignore"):          # exp(-g) = inf for very negative g gives the right limit, -0
                h = g / (1.0 + np.exp(-g)) * u
            if round_h_to is not None:
                h = torch.from_numpy(h).to(torch.float32).to(round_h_to).to(torch.float64).numpy()
            y[t] += w_np[t, k] * (a2 @ h)
    return y


def moe_expected_loops(hidden, w1, w2, ids, wts):
    """Explicit triple-loop float64 statement for tiny shapes (brute force)."""
    x = _f64(hidden)
    a1 = _f64(w1)
    a2 = _f64(w2)
    ids_np = np.asarray(ids).astype(np.int64)
    w_np = _f64(wts)
    n_tok, hdim = x.shape
    inter = a2.shape[-1]
    y = [[0.0] * hdim for _ in range(n_tok)]
    for t in range(n_tok):
        for k in range(ids_np.shape[1]):
            e = int(ids_np[t, k])
            hvec = []
            for j in range(inter):
                g = sum(a1[e, j, c] * x[t, c] for c in range(hdim))
                u = sum(a1[e, inter + j, c] * x[t, c] for c in range(hdim))
                hvec.append(g / (1.0 + np.exp(-g)) * u)
            for r in range(hdim):
                y[t][r] += w_np[t, k] * sum(a2[e, r, j] * hvec[j] for j in range(inter))
    return np.array(y)


def dequant_experts(w_codes, scale):
    """uint8 [E, N, K] + fp32 scale [E, N/128, K/128] -> float32 [E, N, K] holding
    trunc_bf16(e4m3 * scale) (csrc/utils.cuh:80-99; scale shapes
    csrc/moe_kernels/fused_experts_compute.cu:258-266)."""
    w_codes = np.asarray(w_codes, dtype=np.uint8)
    return np.stack([softfp8.dequant_weight_f32(w_codes[e], np.asarray(scale[e], dtype=np.float32))
                     for e in range(w_codes.shape[0])])
