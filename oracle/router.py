"""Router (scores, grouped selection, top-K), restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows csrc/moe_kernels/fused_topK.h (softmax kernel :21-327, sigmoid kernel
:329-607) step by step, one token row at a time, in plain Python:

  scores      softmax: max of the row, exp(x - max), sum, e / sum, rounded to the
              logits dtype T (:74-110); sigmoid: T(1 / (1 + exp(-x))) (:382-386)
  selection   sel = T(p + bias) when a bias is given, else p (:112-131); the
              returned weights are always the un-biased p (:270)
  groups      score of a group = max of sel (no bias) or the sum, in T, of its two
              largest positive sel (bias) (:136-171); keep `topk_group` groups by
              repeated arg-max, ties to the lower group id, a chosen group's score
              is then set to 0 (:172-200); sel and p outside kept groups become 0
              (:202-215)
  top-K       K times: arg-max of sel, ties to the lower expert id, record
              (id, p[id]), set sel[id] = 0 (:226-286)
  order       softmax kernel sorts the K picks by expert id ascending (:294-306);
              the sigmoid kernel leaves them in pick order (:574-586)

Arithmetic definition shared with the HIP kernel so that indices agree bit for
bit: exp, the row sum (index order) and the division are evaluated in float64,
rounded once to fp32 and then to T.  The reference evaluates them with fp32
`expf`; the two differ only where an fp32 rounding straddles a T rounding
boundary, which neither implementation of the reference (device expf vs host
expf) pins either.

Pinned by: brute-force ranking `sorted(range(E), key=(-score, id))[:K]` on
positive scores, rows of equal logits (ids 0..K-1), one-hot logits, and the
library top-k on rows whose K-th and (K+1)-th scores differ.
"""
import numpy as np
import torch


def _round_T(x64, dtype):
    return torch.from_numpy(np.asarray(x64, dtype=np.float64)).to(torch.float32).to(dtype)


def scores(logits, score_fun):
    """[T, E] tensor of dtype T -> probabilities rounded to T (float64 inside)."""
    dtype = logits.dtype
    x = logits.detach().cpu().to(torch.float64).numpy()
    if score_fun == 0:
        mx = x.max(axis=1, keepdims=True)
        e = np.exp(x - mx)
        s = np.zeros(x.shape[0], dtype=np.float64)
        for j in range(x.shape[1]):          # index-order sum
            s = s + e[:, j]
        p = e / s[:, None]
    elif score_fun == 1:
        p = 1.0 / (1.0 + np.exp(-x))
    else:
        raise ValueError("Unsupported scoring function")
    return _round_T(p, dtype)


def route(logits, score_fun, n_groups, topk_groups, topk, bias=None):
    """-> (ids int32 [T, K], weights T [T, K]) exactly as the kernels write them."""
    dtype = logits.dtype
    p_t = scores(logits, score_fun)
    sel_t = p_t if bias is None else (p_t + bias.detach().cpu().to(dtype).reshape(1, -1)).to(dtype)
    p = p_t.to(torch.float64).numpy()
    sel_all = sel_t.to(torch.float64).numpy()
    n_tok, n_exp = p.shape
    per_group = n_exp // n_groups
    ids = np.zeros((n_tok, topk), dtype=np.int32)
    wts = np.zeros((n_tok, topk), dtype=np.float64)

    def add_T(a, b):
        return float(torch.tensor(a, dtype=dtype).add(torch.tensor(b, dtype=dtype)).to(torch.float64))

    for t in range(n_tok):
        sel = sel_all[t].copy()
        prob = p[t].copy()
        # group scores
        gscore = np.zeros(n_groups)
        for g in range(n_groups):
            seg = sel[g * per_group:(g + 1) * per_group]
            if bias is None:
                gscore[g] = max(0.0, seg.max())
            else:
                pos = sorted([v for v in seg if v > 0.0], reverse=True)[:2]
                acc = 0.0
                for v in pos:
                    acc = add_T(v, acc)
                gscore[g] = acc
        kept = []
        work = gscore.copy()
        for _ in range(topk_groups):
            best = 0
            for g in range(1, n_groups):
                if work[g] > work[best]:
                    best = g
            kept.append(best)
            work[best] = 0.0
        for g in range(n_groups):
            if g not in kept:
                sel[g * per_group:(g + 1) * per_group] = 0.0
                prob[g * per_group:(g + 1) * per_group] = 0.0
        # iterative arg-max
        picks = []
        for _ in range(topk):
            best = 0
            for j in range(1, n_exp):
                if sel[j] > sel[best]:
                    best = j
            picks.append((best, prob[best]))
            sel[best] = 0.0
        if score_fun == 0:
            # exchange sort by id as in fused_topK.h:294-306 (stable for distinct ids)
            picks = sorted(picks, key=lambda iw: iw[0])
        for k, (i, w) in enumerate(picks):
            ids[t, k] = i
            wts[t, k] = w
    return torch.from_numpy(ids), torch.from_numpy(wts).to(dtype)


def renormalize(weights):
    """`w / w.sum(-1, keepdim=True)` in the weights' dtype (muxi_moe_planC.py:69-70):
    fp32 sum in index order rounded to T, then each fp32 quotient rounded to T."""
    dtype = weights.dtype
    w32 = weights.to(torch.float32)
    s = torch.zeros(w32.shape[0], dtype=torch.float32)
    for k in range(w32.shape[1]):
        s = s + w32[:, k]
    s = s.to(dtype).to(torch.float32)
    return (w32 / s[:, None]).to(dtype)
