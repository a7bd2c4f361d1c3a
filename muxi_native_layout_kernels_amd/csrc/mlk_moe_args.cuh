// Argument blocks shared by the fused-MoE kernels (mlk_moe.hip, mlk_moe_panel.hip).
#pragma once

#include "mlk_tile.cuh"

namespace mlk {

// One pass over an expert's weights: the token blocks block0 .. block0 + nblocks - 1 of the alignment
// (16 routed pairs each) belong to `expert`.
struct MoeTask {
    int expert, block0, nblocks, pad;
};

struct MoeArgs {
    const uint8_t *W1;        // [E][2I][H] layout-A slabs
    const uint8_t *W2;        // [E][H][I]
    const float *S1;          // [E][2I/128][H/128] or null
    const float *S2;          // [E][H/128][I/128] or null
    const uint16_t *X;        // [T][H]
    uint16_t *Y;              // [T][H]
    uint16_t *Hbuf;           // layout-B [I/32][SB][4][16][8]
    const uint16_t *wts;      // [T*K]
    const int32_t *sorted;    // [T*K + E*15]
    const MoeTask *tasks;
    const int32_t *n_tasks;
    const int32_t *topk_ids;  // [T*K], read by the decode variants that align in-kernel
    const int32_t *experts_map;
    int T, K, H, I, SB, n_pairs, WK, E;
    float *part;              // down projection with K slices: fp32 partial output tiles [slice][workgroup][T][16R]
    int32_t *counters;        // arrival counters, one per down workgroup column (zeroed by the gate/up kernel)
    int n_counters;
};

// Panel kernels for tasks of more than one token block (mlk_moe_panel.cuh): gate/up and down projection of every
// task.  tb32 = blocks of 32 tokens a panel holds (3 or 4), skd = K slices of the down projection; the intermediate
// is kept row-major [slot][I] (slot = position in the alignment), the weighted products go to obuf
// [routed pair][K slice][H] for moe_combine_kernel.  Needs H % 256 == 0.
template <class T, bool FP8>
int launch_moe_panel(const MoeArgs &a, int tb32, int max_tasks, float *obuf, int skd, bool down_pairs, hipStream_t s);

}  // namespace mlk
