// Kernel id 3: panel GeMM for more than 64 tokens over layout-A weights (row-major activations and
// output), where the product is bound by the matrix cores and no longer by the weight stream.
//
// A workgroup of four waves computes a panel of 256 weight rows x 128 tokens over one of SK slices
// of K with v_mfma_f32_32x32x16 (one wave per SIMD issues the 16x16x32 form at little more than half
// rate; the 32x32 form runs at nine tenths of peak from a single wave).  Every wave owns four row
// groups (two pairs of 32 rows) and all four blocks of 32 tokens: eight 32x32 accumulators.  Two other
// shapes exist: 256 rows x 256 tokens (sixteen accumulators, k windows of 64 instead of 128) when that
// makes fewer rounds of one workgroup per CU, and 128 rows x 128 tokens (one pair of row groups per
// wave) while panels are too few to give every CU one.
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
//
// Grid: the token tiles of one row tile run next to each other on one XCD (workgroup id modulo 8
// picks the XCD), so the weights of a row tile are read from HBM once and served to the other token
// tiles by that XCD's L2.  K slices fold like in the row-shared kernel: fp32 partials with
// agent-scope stores, the last workgroup to arrive adds them in slice order.
#include "mlk_panel_loop.cuh"

namespace mlk {

struct PanelArgs {
    const uint8_t *A;
    const uint16_t *B;
    uint16_t *C;
    const uint16_t *bias;
    const float *scale;
    f32x4 *partial;      // [SK][sliced tiles][4 waves][quads of a wave][two planes of 64 x 8 bytes]
    int *counters;       // [sliced tiles], zero between calls
    int M, N, K;
    int SK;              // K slices of the row tiles from whole_groups * 8 on
    int whole_groups;    // groups of eight row tiles in front that are not sliced (0: every row tile has SK slices)
    int row_tiles, token_tiles;
    float alpha;
};

template <class T, bool FP8, int TB, int PR>
__global__ void __launch_bounds__(256, 1) gemm_panel_kernel(PanelArgs p) {
    extern __shared__ u32x4 win[];
    __shared__ int s_last;
    constexpr int R = 2 * PR, KW = panel_kw(TB);               // PR pairs of row groups per wave
    constexpr int WBYTES = FP8 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // workgroup -> (row tile, k slice, token tile): per XCD first the groups of eight row tiles that are computed
    // whole, then the sliced ones
    const int xcd = blockIdx.x & 7;
    int u = blockIdx.x >> 3;
    const int whole_wgs = p.whole_groups * p.token_tiles;
    const bool sliced = u >= whole_wgs;
    const int SK = sliced ? p.SK : 1;
    if (sliced) u -= whole_wgs;
    const int tt = u % p.token_tiles;
    u /= p.token_tiles;
    const int sk = u % SK;
    const int rt = ((sliced ? p.whole_groups : 0) + u / SK) * 8 + xcd;
    if (rt >= p.row_tiles) return;                            // the grid is padded to whole groups of eight row tiles

    const int groups = p.N >> 4;
    const int rg0 = (rt * kTileWaves + wave) * R;
    const int tok0 = tt * (TB * 32);
    const int nwin_total = p.K / (KW * 32);
    const int wbeg = (int)((long long)sk * nwin_total / SK);
    const int nwin = (int)((long long)(sk + 1) * nwin_total / SK) - wbeg;
    const int scale_cols = (p.K + 127) >> 7;

    const uint8_t *abase[R];                                  // wave-uniform; the lane offset is added per load
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int rg = min(rg0 + r, groups - 1);              // rows past N are computed on a copy and never stored
        abase[r] = p.A + (size_t)rg * p.K * 16 * WBYTES;
    }
    ScaleRow srow;
    if (FP8) srow = load_scale_row(p.scale ? p.scale + (size_t)(min(rg0, groups - 1) >> 3) * scale_cols : nullptr, scale_cols, lane);

    // activation staging: a window is 32 TB tokens x GPR granules (k tile colg >> 2, octet colg & 3); granule i of
    // this thread is token trow + RP i of the panel, k granule colg
    constexpr int GPR = KW * 4, RP = 256 / GPR, NG = TB * 32 / RP;
    const int colg = tid % GPR, trow = tid / GPR;
    uint32_t boff[NG];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int tok = min(tok0 + trow + RP * i, p.M - 1);
        boff[i] = (uint32_t)tok * (uint32_t)p.K + colg * 8;
    }
    f32x16 acc[PR][TB];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

    ScaleRow srows[PR];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr) srows[pr] = srow;          // the row groups of a wave lie in one 128-row block
    PanelLoop<T, FP8, TB, PR>::run(acc, abase, srows, p.B, boff, wbeg, nwin, win);

    // accumulator element 4 g + e of lane 32 h + c: weight row 8 g + 4 h + e of the pair's 32, token c of the block's 32
    const int half = lane >> 5, c32 = lane & 31;
    auto epilogue = [&](int pr, int tb, int g, f32x4 v) {
        const int n = (rg0 + 2 * pr) * 16 + 8 * g + 4 * half;
        const int tok = tok0 + tb * 32 + c32;
        if ((n >> 4) >= groups || tok >= p.M) return;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[i] = p.alpha * v[i];
            if (p.bias) o[i] += T::to_f32(p.bias[n + i]);
        }
        store4<T>(p.C + (size_t)tok * p.N + n, o[0], o[1], o[2], o[3]);
    };
    auto quad = [&](const f32x16 &v, int g) { return f32x4{v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]}; };
    if (SK == 1) {
#pragma unroll
        for (int pr = 0; pr < PR; ++pr)
#pragma unroll
            for (int tb = 0; tb < TB; ++tb)
#pragma unroll
                for (int g = 0; g < 4; ++g) epilogue(pr, tb, g, quad(acc[pr][tb], g));
        return;
    }
    const int tile = (rt - p.whole_groups * 8) * p.token_tiles + tt;               // among the sliced tiles
    const int tiles = (p.row_tiles - p.whole_groups * 8) * p.token_tiles;
    // 64-lane group of quad jj of this wave in slice s (two planes of 8-byte halves, see st_agent_planar)
    auto group_at = [&](int s, int jj) -> f32x4 * {
        return p.partial + ((((size_t)s * tiles + tile) * kTileWaves + wave) * (PR * TB * 4) + jj) * 64;
    };
    // partials travel as agent-scope (write-through / always-miss) accesses, like in the narrow kernels; a release /
    // acquire fence pair around ordinary stores was measured slower (it writes back and invalidates a whole L2)
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int g = 0; g < 4; ++g) st_agent_planar(group_at(sk, (pr * TB + tb) * 4 + g), 64, lane, quad(acc[pr][tb], g));
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        int prev = __hip_atomic_fetch_add(&p.counters[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == SK - 1);
        if (s_last) __hip_atomic_store(&p.counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    // slice order; the loads of the next slice are in flight while the current one is added (a round trip to
    // memory per slice would otherwise be paid in full: these loads bypass the caches)
#pragma unroll
    for (int pr = 0; pr < PR; ++pr) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;
        f32x4 t0[TB * 4], t1[TB * 4];
        auto fetch = [&](f32x4 (&t)[TB * 4], int sl) {
#pragma unroll
            for (int jj = 0; jj < TB * 4; ++jj) t[jj] = ld_agent_planar(group_at(sl, pr * TB * 4 + jj), 64, lane);
        };
        auto add = [&](const f32x4 (&t)[TB * 4]) {
#pragma unroll
            for (int tb = 0; tb < TB; ++tb)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[pr][tb][e] += t[tb * 4 + (e >> 2)][e & 3];
        };
        fetch(t0, 0);
        for (int sl = 0; sl < SK; sl += 2) {
            if (sl + 1 < SK) fetch(t1, sl + 1);
            add(t0);
            if (sl + 1 < SK) {
                if (sl + 2 < SK) fetch(t0, sl + 2);
                add(t1);
            }
        }
    }
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int g = 0; g < 4; ++g) epilogue(pr, tb, g, quad(acc[pr][tb], g));
}

// Tokens per panel when the caller leaves the choice open.  Workgroups run one per CU in rounds, and a 256-token
// panel takes 1.84 times as long as a 128-token one (measured), so the width with the cheaper sum of rounds wins.
int panel_tokens(int m, int n) {
    const int cus = device_cus();
    const long long row_tiles = (n + kPanelRowsPerWg - 1) / kPanelRowsPerWg;
    const long long rounds128 = (row_tiles * ((m + 127) / 128) + cus - 1) / cus;
    const long long rounds256 = (row_tiles * ((m + 255) / 256) + cus - 1) / cus;
    return rounds256 * 184 < rounds128 * 100 ? 256 : 128;
}

size_t panel_partial_bytes(int m, int n, int sk) {
    const size_t row_tiles = (n + kPanelRowsPerWg - 1) / kPanelRowsPerWg;
    const size_t tokens = (size_t)((m + 255) / 256) * 256;       // covers both panel widths
    return (size_t)sk * row_tiles * kPanelRowsPerWg * tokens * 4;
}

// a_kind: MLK_F16, MLK_BF16 or MLK_FP8_E4M3 (bf16 activations); width: tokens per panel (128 or 256), anything else =
// panel_tokens(m, n); rows: weight rows per panel (128 or 256; 128 only with 128 tokens), anything else = chosen
// from the number of panels; sk: K slices; last_round_only: slice only the panels that are left over after whole
// rounds of one panel per CU (every panel when there is no whole round, none when nothing is left over)
int launch_panel(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, float alpha, const void *bias,
                 const float *scale, int width, int rows, int sk, bool last_round_only, void *counters,
                 size_t counter_bytes, void *partial, size_t partial_bytes, hipStream_t s) {
    PanelArgs p;
    p.A = (const uint8_t *)a;
    p.B = (const uint16_t *)b;
    p.C = (uint16_t *)c;
    p.bias = (const uint16_t *)bias;
    p.scale = scale;
    p.partial = (f32x4 *)partial;
    p.counters = (int *)counters;
    p.M = m;
    p.N = n;
    p.K = k;
    p.alpha = alpha;
    if (width != 128 && width != 256) width = panel_tokens(m, n);
    p.token_tiles = (m + width - 1) / width;
    MLK_REQUIRE(k % 128 == 0, "gemm: the panel kernel needs K % 128 == 0");
    MLK_REQUIRE((long long)m * k < (1ll << 31), "gemm: the panel kernel indexes activations with 32 bits");
    const int windows = k / (panel_kw(width / 32) * 32);
    if (sk > windows) sk = windows;
    if (sk < 1) sk = 1;
    p.SK = sk;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    if (width == 256) rows = 256;
    if (rows != 128 && rows != 256) {
        const int cus = device_cus();
        // few panels: 128-row panels put twice as many CUs to work (a 128-row panel takes two thirds of the time of
        // a 256-row one); from three eighths of the CU count on, 256-row panels and K slices fill the chip better
        const long long panels256 = (long long)((n + 255) / 256) * p.token_tiles;
        rows = panels256 * 8 <= (long long)cus * 3 ? 128 : 256;
    }
    p.row_tiles = (n + rows - 1) / rows;
    const int groups = (p.row_tiles + 7) / 8;                 // groups of eight row tiles, one per XCD
    p.whole_groups = 0;
    if (last_round_only && sk > 1) {
        // workgroups start in the order of their ids, eight XCDs taking turns: a round is CUs / 8 workgroups per XCD
        const int per_xcd = device_cus() / 8;
        if (p.token_tiles <= per_xcd && per_xcd % p.token_tiles == 0) {
            const int groups_per_round = per_xcd / p.token_tiles;
            p.whole_groups = groups / groups_per_round * groups_per_round;
        }
        if (p.whole_groups == groups) p.whole_groups = 0, p.SK = sk = 1;    // nothing left over
    }
    if (sk > 1) {
        MLK_REQUIRE(partial != nullptr && counters != nullptr, "gemm: a K split across workgroups needs a workspace");
        MLK_REQUIRE((size_t)p.row_tiles * p.token_tiles * sizeof(int) <= counter_bytes,
                    "gemm: too many panels for the counter region");
        if (partial_bytes < panel_partial_bytes(m, n, sk)) return fail(MLK_ERR_WORKSPACE, "gemm: workspace too small");
    }
    const int grid = (p.whole_groups + (groups - p.whole_groups) * sk) * 8 * p.token_tiles;
    // one workgroup per CU (the register ring and the accumulators take a whole SIMD's file); more than 64 KiB of
    // dynamic LDS has to be requested once per kernel
#define MLK_PANEL(TT, F8, TBB, PRR)                                                                                    \
    do {                                                                                                           \
        const size_t lds = (size_t)3 * panel_win(TBB) * 16;                                                        \
        static bool ready_on[64] = {};                           /* the attribute belongs to a device */          \
        bool &ready = ready_on[dev & 63];                                                                          \
        if (!ready) {                                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_panel_kernel<TT, F8, TBB, PRR>),    \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);             \
            if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));                                \
            ready = true;                                                                                          \
        }                                                                                                          \
        gemm_panel_kernel<TT, F8, TBB, PRR><<<grid, 256, lds, s>>>(p);                                                  \
    } while (0)
    if (width == 256) {
        if (a_kind == MLK_FP8_E4M3) MLK_PANEL(BF16, true, 8, 2);
        else if (a_kind == MLK_F16) MLK_PANEL(F16, false, 8, 2);
        else MLK_PANEL(BF16, false, 8, 2);
    } else if (rows == 256) {
        if (a_kind == MLK_FP8_E4M3) MLK_PANEL(BF16, true, 4, 2);
        else if (a_kind == MLK_F16) MLK_PANEL(F16, false, 4, 2);
        else MLK_PANEL(BF16, false, 4, 2);
    } else {
        if (a_kind == MLK_FP8_E4M3) MLK_PANEL(BF16, true, 4, 1);
        else if (a_kind == MLK_F16) MLK_PANEL(F16, false, 4, 1);
        else MLK_PANEL(BF16, false, 4, 1);
    }
#undef MLK_PANEL
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

}  // namespace mlk
