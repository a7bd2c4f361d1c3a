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
#include <type_traits>

#include "mlk_tile.cuh"

namespace mlk {

// Two panel shapes: TB = 4 blocks of 32 tokens (128 tokens, k windows of 128) and TB = 8 (256 tokens, k windows
// of 64).  What a CU can pull through its memory path bounds the kernel once the matrix cores are fed, and a
// 256 x 256 panel moves a third fewer operand bytes per flop than a 256 x 128 one.
constexpr int kPanelRowsPerWg = kTileWaves * 4 * 16;         // 256 rows: two pairs of row groups per wave (128 with one pair)
__host__ __device__ constexpr int panel_kw(int tb) { return tb == 4 ? 4 : 2; }                 // k tiles per window
__host__ __device__ constexpr int panel_tile_stride(int tb) { return tb * 4 * 33 + 4; }         // granules between k tiles
__host__ __device__ constexpr int panel_win(int tb) { return panel_kw(tb) * panel_tile_stride(tb); }

struct PanelArgs {
    const uint8_t *A;
    const uint16_t *B;
    uint16_t *C;
    const uint16_t *bias;
    const float *scale;
    f32x4 *partial;      // [SK][tiles][4 waves][quads of a wave][two planes of 64 x 8 bytes]
    int *counters;       // [tiles], zero between calls
    int M, N, K;
    int SK;
    int row_tiles, token_tiles;
    float alpha;
};

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

template <class T, bool FP8, int TB, int PR>
__global__ void __launch_bounds__(256, 1) gemm_panel_kernel(PanelArgs p) {
    extern __shared__ u32x4 win[];
    __shared__ int s_last;
    constexpr int R = 2 * PR, KW = panel_kw(TB), WG = panel_win(TB), TS = panel_tile_stride(TB);   // PR pairs of row groups per wave
    constexpr int WBYTES = FP8 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // workgroup -> (row tile, k slice, token tile)
    const int xcd = blockIdx.x & 7;
    int u = blockIdx.x >> 3;
    const int tt = u % p.token_tiles;
    u /= p.token_tiles;
    const int sk = u % p.SK;
    const int rt = (u / p.SK) * 8 + xcd;
    if (rt >= p.row_tiles) return;                            // the grid is padded to whole groups of eight row tiles

    const int groups = p.N >> 4;
    const int rg0 = (rt * kTileWaves + wave) * R;
    const int tok0 = tt * (TB * 32);
    const int nwin_total = p.K / (KW * 32);
    const int wbeg = (int)((long long)sk * nwin_total / p.SK);
    const int nwin = (int)((long long)(sk + 1) * nwin_total / p.SK) - wbeg;
    const int scale_cols = (p.K + 127) >> 7;

    const uint8_t *abase[R];                                  // wave-uniform; the lane offset is added per load
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int rg = min(rg0 + r, groups - 1);              // rows past N are computed on a copy and never stored
        abase[r] = p.A + (size_t)rg * p.K * 16 * WBYTES;
    }
    const uint32_t lane_off = lane * (FP8 ? 8 : 16);
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
    const int st_idx = (colg >> 2) * TS + (colg & 3) * 33 + trow;             // + st_off(i)
    auto st_off = [](int i) { return ((RP * i) / 32) * 4 * 33 + (RP * i) % 32; };
    const int ld_idx = (lane >> 5) * 33 + (lane & 31);                        // + t * TS + (tb * 4 + 2 s) * 33

    f32x16 acc[PR][TB];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

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
        for (int i = 0; i < NG; ++i) br[i] = ld_global_u32x4(p.B + boff[i] + k0);
    };
    auto stage_store = [&](const u32x4 (&br)[NG], int base) {
#pragma unroll
        for (int i = 0; i < NG; ++i) win[base + st_idx + st_off(i)] = br[i];
    };
    WeightFrag<FP8> wf[2][KW][R];
    float sc[2];                                              // a window lies inside one 128-wide scale block
    auto issue_a = [&](int slot, int w, int t) {              // tile t of window w
        const int tile = (wbeg + w) * KW + t;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if constexpr (FP8) wf[slot][t][r].v = *reinterpret_cast<const u32x2 *>(abase[r] + (size_t)tile * 512 + lane_off);
            else wf[slot][t][r].v = ld_global_u32x4(abase[r] + (size_t)tile * 1024 + lane_off);
        }
        if (FP8 && t == KW - 1) sc[slot] = scale_at(srow, tile >> 2);   // after the last use of the slot's previous scale
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
        for (int r = 0; r < R; ++r) s4[r] = FP8 ? sc[slot] : 1.f;
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
    if (p.SK == 1) {
#pragma unroll
        for (int pr = 0; pr < PR; ++pr)
#pragma unroll
            for (int tb = 0; tb < TB; ++tb)
#pragma unroll
                for (int g = 0; g < 4; ++g) epilogue(pr, tb, g, quad(acc[pr][tb], g));
        return;
    }
    const int tile = rt * p.token_tiles + tt;
    const int tiles = p.row_tiles * p.token_tiles;
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
        s_last = (prev == p.SK - 1);
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
        for (int sl = 0; sl < p.SK; sl += 2) {
            if (sl + 1 < p.SK) fetch(t1, sl + 1);
            add(t0);
            if (sl + 1 < p.SK) {
                if (sl + 2 < p.SK) fetch(t0, sl + 2);
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
// from the number of panels
int launch_panel(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, float alpha, const void *bias,
                 const float *scale, int width, int rows, int sk, void *counters, size_t counter_bytes, void *partial,
                 size_t partial_bytes, hipStream_t s) {
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
    if (sk > 1) {
        MLK_REQUIRE(partial != nullptr && counters != nullptr, "gemm: a K split across workgroups needs a workspace");
        MLK_REQUIRE((size_t)p.row_tiles * p.token_tiles * sizeof(int) <= counter_bytes,
                    "gemm: too many panels for the counter region");
        if (partial_bytes < panel_partial_bytes(m, n, sk)) return fail(MLK_ERR_WORKSPACE, "gemm: workspace too small");
    }
    const int grid = ((p.row_tiles + 7) / 8) * 8 * p.token_tiles * sk;
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
