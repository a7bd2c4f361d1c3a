// Main loop of the panel kernels: a workgroup of four waves multiplies a panel of weight rows (each wave PR pairs
// of row groups, 32 rows per pair) with TB blocks of 32 token rows over a run of k windows, with
// v_mfma_f32_32x32x16.  Used by the panel GeMM (mlk_panel.hip) and by the fused MoE above 16 tokens per expert
// (mlk_moe_panel.hip), which differ in where the rows come from and in what happens to the accumulators.
//
// Weights come straight from global memory, two k windows ahead in a register ring.  A layout-A
// tile (16 rows x 32 k: lane 16 q + r holds row r, k octet q) is not the 32x32x16 operand (lane
// 32 g + i holds row i, k octet g of a 16-wide k slice), but two vertically adjacent tiles X, Y become
// the two operands of their 32 k with two lane swaps per register: v_permlane16_swap turns the
// 16-lane rows [X0 X1 X2 X3], [Y0 Y1 Y2 Y3] into [X0 Y0 X2 Y2], [X1 Y1 X3 Y3], v_permlane32_swap
// then into [X0 Y0 X1 Y1] (k octets 0, 1 of rows 0..31) and [X2 Y2 X3 Y3] (octets 2, 3).
//
// The activations of a k window are fetched once per workgroup with 16-byte loads two windows ahead
// (they wait in registers) and parked in LDS one window ahead in operand order: granule
// ((t*TB + tb)*4 + octet)*33 + token (+ 4 t) for k tile t, token block tb, so that an operand is two
// runs of 32 consecutive granules for ds_read_b128 and the granules a token row contributes fall into
// different banks.  Three LDS buffers, one barrier per window; within a window the LDS reads and the
// global loads are scheduled between the MFMAs (sched_group_barrier).
#pragma once

#include <type_traits>

#include "mlk_tile.cuh"

namespace mlk {

// Two panel shapes: TB = 4 blocks of 32 tokens (128 tokens, k windows of 128) and TB = 8 (256 tokens, k windows
// of 64).  What a CU can pull through its memory path bounds the kernel once the matrix cores are fed, and a
// 256 x 256 panel moves a third fewer operand bytes per flop than a 256 x 128 one.
constexpr int kPanelRowsPerWg = kTileWaves * 4 * 16;         // 256 rows: two pairs of row groups per wave (128 with one pair)
__host__ __device__ constexpr int panel_kw(int tb) { return tb <= 4 ? 4 : 2; }                 // k tiles per window
__host__ __device__ constexpr int panel_tile_stride(int tb) { return tb * 4 * 33 + 4; }         // granules between k tiles
__host__ __device__ constexpr int panel_win(int tb) { return panel_kw(tb) * panel_tile_stride(tb); }


// LDS bytes of a panel workgroup: three activation windows
__host__ __device__ constexpr size_t panel_lds_bytes(int tb) { return (size_t)3 * panel_win(tb) * 16; }
// 16-byte granules of an activation window that one thread moves, and the token rows between them
__host__ __device__ constexpr int panel_rp(int tb) { return 256 / (panel_kw(tb) * 4); }
__host__ __device__ constexpr int panel_ng(int tb) { return tb * 32 / panel_rp(tb); }

// Two vertically adjacent layout-A fragments -> the 32x32x16 operands of k octets {0, 1} (in x) and {2, 3} (in y).
__device__ __forceinline__ void pair_to_rows32(u32x4 &x, u32x4 &y) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        auto s16 = __builtin_amdgcn_permlane16_swap(x[d], y[d], false, false);
        auto s32 = __builtin_amdgcn_permlane32_swap(s16[0], s16[1], false, false);
        x[d] = s32[0];
        y[d] = s32[1];
    }
}

// acc[pr][tb] += rows of pair pr x the tokens of block tb, over the windows wbeg .. wbeg + nwin - 1 of KW k tiles.
//   abase[r]   wave-uniform start of row group r of this wave (r = 2 pr, 2 pr + 1 form pair pr)
//   srow[pr]   soft-FP8 block scales of the 128-row block that holds pair pr
//   B, boff[i] the thread's granule i of an activation window comes from B + boff[i] + (first k of the window):
//              token row trow + RP i of the panel (trow = tid / (4 KW)), k granule tid % (4 KW)
//   win        3 * panel_win(TB) granules of LDS
template <class T, bool FP8, int TB, int PR>
struct PanelLoop {
    static constexpr int R = 2 * PR, KW = panel_kw(TB), WG = panel_win(TB), TS = panel_tile_stride(TB);
    static constexpr int GPR = KW * 4, RP = 256 / GPR, NG = TB * 32 / RP;

    __device__ static __forceinline__ void run(f32x16 (&acc)[PR][TB], const uint8_t *const (&abase)[R],
                                               const ScaleRow (&srow)[PR], const uint16_t *__restrict__ B,
                                               const uint32_t (&boff)[NG], int wbeg, int nwin, u32x4 *win) {
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t lane_off = lane * (FP8 ? 8 : 16);
    const int colg = tid % GPR, trow = tid / GPR;
    const int st_idx = (colg >> 2) * TS + (colg & 3) * 33 + trow;             // + st_off(i)
    auto st_off = [](int i) { return ((RP * i) / 32) * 4 * 33 + (RP * i) % 32; };
    const int ld_idx = (lane >> 5) * 33 + (lane & 31);                        // + t * TS + (tb * 4 + 2 s) * 33

    // Pipeline of one window j (128 k; weight slot j & 1, LDS buffer j % 3) in eight half steps of eight
    // MFMAs (16 k x four token blocks x two row pairs).  While a half step multiplies out of one set of
    // fragment registers the LDS reads of the next half step land in the other set.  Everything that
    // comes from memory is requested well before it is used: the weights of tile t of window j + 2
    // once tile t of window j has been multiplied (same registers), the activations of window
    // j + 2 at the start of window j; they are written to LDS in the middle of window j + 1 and
    // published by the single barrier there, so that the reads of the first half step of window
    // j + 2 can go out during the last half step of window j + 1.  With three LDS buffers that one
    // barrier per window is enough: the buffer written in the middle of window j was last read in
    // window j - 2, which every wave has left before it reaches the barrier of window j - 1.
    u32x4 bring[2][NG];                                       // window w travels in bring[w & 1]
    auto stage_load = [&](u32x4 (&br)[NG], int w) {           // window index inside the slice
        const size_t k0 = (size_t)(wbeg + w) * (KW * 32);
#pragma unroll
        for (int i = 0; i < NG; ++i) br[i] = ld_global_u32x4(B + boff[i] + k0);
    };
    auto stage_store = [&](const u32x4 (&br)[NG], int base) {
#pragma unroll
        for (int i = 0; i < NG; ++i) win[base + st_idx + st_off(i)] = br[i];
    };
    WeightFrag<FP8> wf[2][KW][R];
    float sc[2][PR];                                          // a window lies inside one 128-wide scale block; one scale per row pair
    auto issue_a = [&](int slot, int w, int t) {              // tile t of window w
        const int tile = (wbeg + w) * KW + t;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if constexpr (FP8) wf[slot][t][r].v = *reinterpret_cast<const u32x2 *>(abase[r] + (size_t)tile * 512 + lane_off);
            else wf[slot][t][r].v = ld_global_u32x4(abase[r] + (size_t)tile * 1024 + lane_off);
        }
        if (FP8 && t == KW - 1) {                             // after the last use of the slot's previous scales
#pragma unroll
            for (int pr = 0; pr < PR; ++pr) sc[slot][pr] = scale_at(srow[pr], tile >> 2);
        }
    };
    u32x4 b0[TB], b1[TB];
    auto rd = [&](u32x4 (&b)[TB], int base, int t, int s) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            b[tb] = win[base + t * TS + (tb * 4 + 2 * s) * 33 + ld_idx];
        }
    };
    // a[2 pr + s]: row pair pr, k half s
    auto mm = [&](const u32x4 (&a)[R], const u32x4 (&b)[TB], int s) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int pr = 0; pr < PR; ++pr) {
                acc[pr][tb] = T::mfma32(a[2 * pr + s], b[tb], acc[pr][tb]);
            }
    };
    auto operands = [&](u32x4 (&a)[R], int slot, int t) {
        float s4[R];
#pragma unroll
        for (int r = 0; r < R; ++r) s4[r] = FP8 ? sc[slot][r >> 1] : 1.f;
        weight_operands<FP8, R>(a, wf[slot][t], s4);
        pair_to_rows32(a[0], a[1]);
        if constexpr (PR == 2) pair_to_rows32(a[2], a[3]);
    };
    int cur = 0;                                              // LDS granule offset of the current window's buffer
    // SLOT: weight slot; NEXT / NEXT2: windows j + 1 / j + 2 exist (compile-time, so the steady loop has no tests)
    auto window = [&](auto slot_c, auto next_c, auto next2_c, int j) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr bool NEXT = decltype(next_c)::value, NEXT2 = decltype(next2_c)::value;
        const int nxt = cur == 2 * WG ? 0 : cur + WG;
        u32x4 a[R];
        auto half = [&](auto hs_c, const u32x4 (&use)[TB], u32x4 (&other)[TB]) {
            constexpr int hs = decltype(hs_c)::value, t = hs >> 1, sh = hs & 1;
            if (sh == 0) operands(a, slot, t);
            if (hs < 2 * KW - 1) rd(other, cur, (hs + 1) >> 1, (hs + 1) & 1);
            else if (NEXT) rd(other, nxt, 0, 0);
            if (hs == 0 && NEXT2) stage_load(bring[slot], j + 2);
            if (sh == 0 && t > 0 && NEXT2) issue_a(slot, j + 2, t - 1);   // the registers of tile t - 1 are free again
            mm(a, use, sh);
            // one scheduling region: the LDS reads and global loads above go out between the MFMAs
#pragma unroll
            for (int i = 0; i < TB; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // global load
            }
            __builtin_amdgcn_sched_barrier(0);
            if (hs == 2 * KW - 1 && NEXT2) issue_a(slot, j + 2, KW - 1);
            if (hs == KW - 1) {
                if (NEXT) stage_store(bring[slot ^ 1], nxt);
                __syncthreads();
            }
        };
        half(std::integral_constant<int, 0>{}, b0, b1);
        half(std::integral_constant<int, 1>{}, b1, b0);
        half(std::integral_constant<int, 2>{}, b0, b1);
        half(std::integral_constant<int, 3>{}, b1, b0);
        if constexpr (KW == 4) {
            half(std::integral_constant<int, 4>{}, b0, b1);
            half(std::integral_constant<int, 5>{}, b1, b0);
            half(std::integral_constant<int, 6>{}, b0, b1);
            half(std::integral_constant<int, 7>{}, b1, b0);
        }
        cur = nxt;
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using Yes = std::true_type;
    using No = std::false_type;

    if (nwin > 0) {
        stage_load(bring[0], 0);
#pragma unroll
        for (int t = 0; t < KW; ++t) issue_a(0, 0, t);
        stage_store(bring[0], 0);
        if (nwin > 1) {
            stage_load(bring[1], 1);
#pragma unroll
            for (int t = 0; t < KW; ++t) issue_a(1, 1, t);
        }
        __syncthreads();
        rd(b0, 0, 0, 0);
        int j = 0;
        for (; j + 3 < nwin; j += 2) {
            window(I0{}, Yes{}, Yes{}, j);
            window(I1{}, Yes{}, Yes{}, j + 1);
        }
        const int rem = nwin - j;                             // 1, 2 or 3
        if (rem == 3) {
            window(I0{}, Yes{}, Yes{}, j);
            window(I1{}, Yes{}, No{}, j + 1);
            window(I0{}, No{}, No{}, j + 2);
        } else if (rem == 2) {
            window(I0{}, Yes{}, No{}, j);
            window(I1{}, No{}, No{}, j + 1);
        } else {
            window(I0{}, No{}, No{}, j);
        }
    }
    mfma_settle();
    }
};

}  // namespace mlk
