// Fused MoE above 16 tokens per expert on the LDS-fed panel main loop (PanelLoopLds, mlk_panel_lds.cuh):
// v_mfma_f32_32x32x16, weights from the per-expert layout-A slabs straight into an LDS ring, the task's token rows
// shared through the same ring.
//
//   gate/up   grid (I / 128, tasks).  A wave owns 32 columns of the intermediate: one pair of row groups from the
//             gate half of W1[expert] and the pair with the same index from the up half, so that gate and up of an
//             element sit in the same accumulator slot and SiLU(gate) * up needs no exchange.  The token rows are
//             gathered through the alignment (`sorted`), TB blocks of 32 per panel.  The result goes to the
//             intermediate buffer row-major, one row of I per slot of the alignment.
//   down      grid (H / 256, tasks, K slices).  A wave owns two pairs of row groups of W2[expert]; the activations
//             are the task's rows of the intermediate.  Products times the routing weight go to an fp32 buffer
//             per (routed pair, K slice); moe_combine_kernel adds them per token in pick order.
//
// Slots of a task that hold no routed pair (padding of the last 16-slot block, or blocks beyond the task) read some
// valid row and are never stored: a column of the product depends only on its own token row.
//
// Where it is used: soft-FP8 weights with more than 64 tokens per pass over an expert.  There the weight stream is
// half as long as with 16-bit weights and the matrix cores set the pace; the row-shared kernels (16x16x32
// products, one wave per SIMD) reach about a fifth of their peak, this loop about two fifths (measured on the
// Mixtral shape at 256 tokens: 549 us -> 385 us).  With 16-bit weights, and with fewer tokens per expert, the layer
// is bound by the weight stream and the row-shared kernels are as fast or faster (measured with this loop on bf16
// weights: gate/up 362 against 325 us), so only the soft-FP8 form is instantiated (mlk_moe_panel_fp8.hip).
#pragma once

#include "mlk_moe_args.cuh"
#include "mlk_panel_lds.cuh"

namespace mlk {

// Slabs of LDS per workgroup.  Gate/up: four (56 or 64 KiB), two workgroups per CU.  Down: the same where the host
// found a K split that fills two workgroups per CU (moe_panel_down_shape in mlk_moe.hip), else six (84 or 96 KiB),
// which keeps it to one workgroup per CU: on a grid of about one workgroup per CU, two of them on one CU while
// another CU idles cost more than the second wave per SIMD brings (Mixtral shape, 256 tokens, 2 K slices: 177
// against 137 us; 4 K slices on the short ring: 117 us).
constexpr int kMoeGateUpRing = 4, kMoeDownRing = 6, kMoeDownPairRing = 4;

template <class T, bool FP8, int TB>
__global__ void __launch_bounds__(256, 2) moe_gate_up_panel_kernel(MoeArgs p) {
    extern __shared__ u32x4 win[];
    const int task = blockIdx.y;
    if (task >= p.n_tasks[0]) return;
    const MoeTask tk = p.tasks[task];
    using Loop = PanelLoopLds<T, FP8, TB, kMoeGateUpRing>;
    constexpr int WB = FP8 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col0 = (blockIdx.x * kTileWaves + wave) * 32;       // first of the wave's 32 intermediate columns
    const int groups_i = p.I >> 4;
    const size_t slab = (size_t)2 * p.I * p.H * WB;
    const int scale_cols = p.H >> 7;

    const uint8_t *abase[4];
    ScaleRow srow[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {                       // 0: gate rows, 1: up rows
        const int rg = half * groups_i + (col0 >> 4);
#pragma unroll
        for (int r = 0; r < 2; ++r) abase[2 * half + r] = p.W1 + (size_t)tk.expert * slab + (size_t)(rg + r) * p.H * 16 * WB;
        if (FP8)
            srow[half] = load_scale_row(p.S1 ? p.S1 + ((size_t)tk.expert * (2 * p.I >> 7) + (rg >> 3)) * scale_cols : nullptr,
                                        scale_cols, lane);
    }
    const int slots = tk.nblocks * 16;
    auto row_off = [&](int slot) -> uint32_t {                 // the token row that slot `slot` of the task reads
        int id = p.n_pairs;
        if (slot < slots) id = p.sorted[tk.block0 * 16 + slot];
        const int tok = id < p.n_pairs ? id / p.K : 0;
        return (uint32_t)tok * (uint32_t)p.H;
    };
    f32x16 acc[2][TB];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

    Loop::run(acc, abase, srow, p.X, row_off, 0, p.H >> 5, win);

    // accumulator element 4 g + e of lane 32 h + c: row 8 g + 4 h + e of the pair's 32, token c of the block's 32
    const int half = lane >> 5, c32 = lane & 31;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        const int slot = tb * 32 + c32;
        if (slot >= slots) continue;
        if (p.sorted[tk.block0 * 16 + slot] >= p.n_pairs) continue;
        uint16_t *row = p.Hbuf + (size_t)(tk.block0 * 16 + slot) * p.I + col0 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float gate = acc[0][tb][4 * g + e], up = acc[1][tb][4 * g + e];
                h[e] = gate / (1.f + __expf(-gate)) * up;
            }
            store4<T>(row + 8 * g, h[0], h[1], h[2], h[3]);
        }
    }
}

template <class T, bool FP8, int TB, int RING>
__global__ void __launch_bounds__(256, 2) moe_down_panel_kernel(MoeArgs p, float *__restrict__ O) {
    extern __shared__ u32x4 win[];
    const int task = blockIdx.y;
    if (task >= p.n_tasks[0]) return;
    const MoeTask tk = p.tasks[task];
    using Loop = PanelLoopLds<T, FP8, TB, RING>;
    constexpr int WB = FP8 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg0 = (blockIdx.x * kTileWaves + wave) * 4;          // four row groups = 64 output rows per wave
    const size_t slab = (size_t)p.H * p.I * WB;
    const int scale_cols = p.I >> 7;

    const uint8_t *abase[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) abase[r] = p.W2 + (size_t)tk.expert * slab + (size_t)(rg0 + r) * p.I * 16 * WB;
    ScaleRow srow[2];
    if (FP8) {
        srow[0] = load_scale_row(p.S2 ? p.S2 + ((size_t)tk.expert * (p.H >> 7) + (rg0 >> 3)) * scale_cols : nullptr, scale_cols, lane);
        srow[1] = srow[0];                                         // 64 rows from a multiple of 64: one 128-row block
    }
    const int slots = tk.nblocks * 16;
    auto row_off = [&](int slot) -> uint32_t {                 // rows of the intermediate, one per slot of the alignment
        return (uint32_t)(tk.block0 * 16 + (slot < slots ? slot : 0)) * (uint32_t)p.I;
    };
    f32x16 acc[2][TB];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

    const int nwin_total = p.I >> 7;                              // K slices are cut at multiples of 128 k
    const int wbeg = (int)((long long)blockIdx.z * nwin_total / (int)gridDim.z);
    const int nwin = (int)((long long)(blockIdx.z + 1) * nwin_total / (int)gridDim.z) - wbeg;
    Loop::run(acc, abase, srow, p.Hbuf, row_off, 4 * wbeg, 4 * nwin, win);

    const int half = lane >> 5, c32 = lane & 31;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        const int slot = tb * 32 + c32;
        if (slot >= slots) continue;
        const int id = p.sorted[tk.block0 * 16 + slot];
        if (id >= p.n_pairs) continue;
        const float wt = T::to_f32(p.wts[id]);
        float *row = O + ((size_t)id * gridDim.z + blockIdx.z) * p.H + rg0 * 16 + 4 * half;
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {acc[pr][tb][4 * g], acc[pr][tb][4 * g + 1], acc[pr][tb][4 * g + 2], acc[pr][tb][4 * g + 3]};
                v *= wt;
                *reinterpret_cast<f32x4 *>(row + pr * 32 + 8 * g) = v;
            }
    }
}

// More than 64 KiB of dynamic LDS has to be allowed once per kernel and device.
template <class K>
static int panel_lds_attribute(K kernel, size_t lds, bool (&ready_on)[64]) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    bool &ready = ready_on[dev & 63];
    if (!ready && lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));
    }
    ready = true;
    return MLK_OK;
}

template <class T, bool FP8, int TB>
static int launch_moe_panel_tb(const MoeArgs &a, int max_tasks, float *obuf, int skd, bool down_pairs, hipStream_t s) {
    const size_t lds = PanelLdsShape<FP8, TB, kMoeGateUpRing>::lds_bytes;
    const size_t lds_down = PanelLdsShape<FP8, TB, kMoeDownRing>::lds_bytes;
    const size_t lds_down2 = PanelLdsShape<FP8, TB, kMoeDownPairRing>::lds_bytes;
    static bool ready_gate[64] = {}, ready_down[64] = {}, ready_down2[64] = {};
    int rc = panel_lds_attribute(&moe_gate_up_panel_kernel<T, FP8, TB>, lds, ready_gate);
    if (rc != MLK_OK) return rc;
    rc = panel_lds_attribute(&moe_down_panel_kernel<T, FP8, TB, kMoeDownRing>, lds_down, ready_down);
    if (rc != MLK_OK) return rc;
    rc = panel_lds_attribute(&moe_down_panel_kernel<T, FP8, TB, kMoeDownPairRing>, lds_down2, ready_down2);
    if (rc != MLK_OK) return rc;
    moe_gate_up_panel_kernel<T, FP8, TB><<<dim3(a.I / 128, max_tasks), 256, lds, s>>>(a);
    MLK_LAUNCH_CHECK();
    if (down_pairs)
        moe_down_panel_kernel<T, FP8, TB, kMoeDownPairRing><<<dim3(a.H / 256, max_tasks, skd), 256, lds_down2, s>>>(a, obuf);
    else
        moe_down_panel_kernel<T, FP8, TB, kMoeDownRing><<<dim3(a.H / 256, max_tasks, skd), 256, lds_down, s>>>(a, obuf);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

template <class T, bool FP8>
int launch_moe_panel(const MoeArgs &a, int tb32, int max_tasks, float *obuf, int skd, bool down_pairs, hipStream_t s) {
    switch (tb32) {
        case 3: return launch_moe_panel_tb<T, FP8, 3>(a, max_tasks, obuf, skd, down_pairs, s);
        case 4: return launch_moe_panel_tb<T, FP8, 4>(a, max_tasks, obuf, skd, down_pairs, s);
        default: return fail(MLK_ERR_INVALID, "moe: a panel holds 3 or 4 blocks of 32 tokens");
    }
}

}  // namespace mlk
