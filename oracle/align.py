"""Token -> expert-block alignment (the MoE permutation), restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows csrc/moe_kernels/moe_align_tokens.h:8-94 (counts, padding to the block
size, inclusive scan, block owners) and moe_align_tokens.cu:5-21 (scatter of the
flat pair indices).  The reference's scatter takes its slot from an atomic
cursor, so the order inside one expert's segment is whatever the hardware
schedules; this statement fixes it to ascending flat index, which is one of the
orders the reference can produce.

Pinned by invariants (every routed pair appears exactly once inside its
expert's segment, segments start at multiples of the block size in expert
order, pad slots hold the sentinel, block owners, padded block count) and by
brute force on the 64-entry example the reference holds
(csrc/moe_kernels/test_moe_align_tokens.cc:12-16).
"""
import numpy as np


def align_tokens(topk_ids, num_experts, block=16, experts_map=None):
    """topk_ids: int array [T, K] (or flat).  Returns a dict with

    sorted_token_ids   int32 [T*K + E*(block-1)], sentinel T*K in unused slots
                       (pre-filled by the caller, muxi_moe_planC.py:82-88)
    cumsum             int32 [E+1], padded inclusive prefix BEFORE the scatter
                       (moe_align_tokens.h:57-79,87)
    cursors            int32 [E+1], what the reference leaves in cumsum_buffer
                       after the scatter: cumsum[e] + count[e] for e < E
    padded_num_blocks  int, cumsum[E] / block (moe_align_tokens.h:80-82)
    experts_ids        int32 [ceil((T*K + E*(block-1)) / block)], owner of each
                       block, 0 elsewhere (:31-33, :88-92)
    counts             int32 [E]
    """
    flat = np.asarray(topk_ids, dtype=np.int64).reshape(-1)
    numel = flat.size
    max_padded = numel + num_experts * (block - 1)
    counts = np.zeros(num_experts, dtype=np.int64)
    local = np.empty(numel, dtype=np.int64)
    for i, e in enumerate(flat):
        le = int(e) if experts_map is None else int(experts_map[int(e)])
        local[i] = le
        if le != -1:
            counts[le] += 1
    padded = (counts + block - 1) // block * block
    cumsum = np.zeros(num_experts + 1, dtype=np.int64)
    for e in range(num_experts):
        cumsum[e + 1] = cumsum[e] + padded[e]
    experts_ids = np.zeros((max_padded + block - 1) // block, dtype=np.int32)
    for e in range(num_experts):
        for s in range(cumsum[e], cumsum[e + 1], block):
            experts_ids[s // block] = e
    sorted_ids = np.full(max_padded, numel, dtype=np.int32)
    cursor = cumsum.copy()
    for i in range(numel):            # ascending flat index inside each expert
        le = local[i]
        if le == -1:
            continue
        sorted_ids[cursor[le]] = i
        cursor[le] += 1
    return dict(sorted_token_ids=sorted_ids, cumsum=cumsum.astype(np.int32),
                cursors=cursor.astype(np.int32), padded_num_blocks=int(cumsum[-1] // block),
                experts_ids=experts_ids, counts=counts.astype(np.int32))
