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
#include "mlk_panel_lds.cuh"

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
    int band, chunk;     // gemm_panel8_kernel: groups of row tiles and token tiles that neighbouring workgroups of an XCD cover
    float alpha;
};

// What happens to the accumulators of a panel: scaled and stored, or (K slices) handed over as fp32 partials that the
// last workgroup to arrive adds in slice order.  acc[pr][tb] covers the row groups rg0 + 2 pr, + 1 and the 32 tokens from
// tok0 + 32 tb on; NWAVES waves per workgroup, each with PR x TB accumulators; the fold fetches FB accumulators at a time.
template <class T, int PR, int TB, int NWAVES, int FB>
__device__ __forceinline__ void panel_finish(const PanelArgs &p, f32x16 (&acc)[PR][TB], int rg0, int tok0, int SK, int sk,
                                             int rt, int tt, int wave, int lane, int *s_last) {
    const int groups = p.N >> 4;
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
        return p.partial + ((((size_t)s * tiles + tile) * NWAVES + wave) * (PR * TB * 4) + jj) * 64;
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
        *s_last = (prev == SK - 1);
        if (*s_last) __hip_atomic_store(&p.counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!*s_last) return;
    // slice order; the loads of the next slice are in flight while the current one is added (a round trip to
    // memory per slice would otherwise be paid in full: these loads bypass the caches).  FB accumulators are fetched
    // at a time: all of a row pair's where the registers allow it.
    static_assert(TB % FB == 0, "fetch groups are whole accumulators of one row pair");
#pragma unroll
    for (int pr = 0; pr < PR; ++pr) {
#pragma unroll
        for (int t0b = 0; t0b < TB; t0b += FB) {
#pragma unroll
            for (int tb = 0; tb < FB; ++tb)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[pr][t0b + tb][e] = 0.f;
            f32x4 t0[FB * 4], t1[FB * 4];
            auto fetch = [&](f32x4 (&t)[FB * 4], int sl) {
#pragma unroll
                for (int jj = 0; jj < FB * 4; ++jj) t[jj] = ld_agent_planar(group_at(sl, (pr * TB + t0b) * 4 + jj), 64, lane);
            };
            auto add = [&](const f32x4 (&t)[FB * 4]) {
#pragma unroll
                for (int tb = 0; tb < FB; ++tb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[pr][t0b + tb][e] += t[tb * 4 + (e >> 2)][e & 3];
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
    }
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int g = 0; g < 4; ++g) epilogue(pr, tb, g, quad(acc[pr][tb], g));
}

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

    panel_finish<T, PR, TB, kTileWaves, TB>(p, acc, rg0, tok0, SK, sk, rt, tt, wave, lane, &s_last);
}

// 256 x 128 panels on the loop of mlk_panel_lds.cuh (four waves, LDS as the prefetch buffer; soft-FP8: two workgroups
// per CU).  Same grid and fold as gemm_panel_kernel.
template <class T, bool FP8, int RING>
__global__ void __launch_bounds__(256, 2) gemm_panel_lds_kernel(PanelArgs p) {
    extern __shared__ u32x4 win[];
    constexpr int TB = 4, PR = 2, R = 4;
    constexpr int WBYTES = FP8 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    if (rt >= p.row_tiles) return;

    const int groups = p.N >> 4;
    const int rg0 = (rt * kTileWaves + wave) * R;
    const int tok0 = tt * (TB * 32);
    const int nwin_total = p.K / 128;                          // slices are cut in windows of 128 k, as the host counts them
    const int wbeg = (int)((long long)sk * nwin_total / SK);
    const int nwin = (int)((long long)(sk + 1) * nwin_total / SK) - wbeg;
    const int scale_cols = (p.K + 127) >> 7;
    const uint8_t *abase[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int rg = min(rg0 + r, groups - 1);              // rows past N are computed on a copy and never stored
        abase[r] = p.A + (size_t)rg * p.K * 16 * WBYTES;
    }
    ScaleRow srows[PR];
    if (FP8) {
        srows[0] = load_scale_row(p.scale ? p.scale + (size_t)(min(rg0, groups - 1) >> 3) * scale_cols : nullptr, scale_cols, lane);
        srows[1] = srows[0];                                   // the row groups of a wave lie in one 128-row block
    }
    auto row_off = [&](int slot) -> uint32_t { return (uint32_t)min(tok0 + slot, p.M - 1) * (uint32_t)p.K; };
    f32x16 acc[PR][TB];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;
    PanelLoopLds<T, FP8, TB, RING>::run(acc, abase, srows, p.B, row_off, 4 * wbeg, 4 * nwin, win);
    __syncthreads();                                           // the ring is given up: its first word takes the fold's flag
    panel_finish<T, PR, TB, kTileWaves, 2>(p, acc, rg0, tok0, SK, sk, rt, tt, wave, lane, reinterpret_cast<int *>(win));
}

// Output of an eight-wave panel that is computed whole: every wave turns its 64 rows x 128 tokens around in LDS (the ring
// is free by then; 144 bytes per token, so that the 8-byte pieces of 32 tokens meet each bank at most twice) and stores
// whole 128-byte lines, eight tokens per instruction.  Stored straight from the accumulators, a lane's four rows of one
// token are 8 bytes in a line that fifteen other instructions complete: 67 MB of output took 23 us that way.
constexpr int kP8OutPitch = 144;                               // bytes per token in the turn-around buffer
constexpr size_t kP8OutBytes = (size_t)8 * 128 * kP8OutPitch;
template <class T>
__device__ __forceinline__ void p8_store_panel(const PanelArgs &p, f32x16 (&acc)[2][4], int rg0, int tok0, int wave, int lane,
                                               u32x4 *win) {
    uint8_t *buf = reinterpret_cast<uint8_t *>(win) + (size_t)wave * 128 * kP8OutPitch;
    const int half = lane >> 5, c32 = lane & 31;
    const int n0 = rg0 * 16;                                   // first of the wave's 64 rows
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int row = pr * 32 + 8 * g + 4 * half;        // of the wave's 64
            float bias[4] = {0.f, 0.f, 0.f, 0.f};
            if (p.bias && n0 + row < p.N) {
#pragma unroll
                for (int i = 0; i < 4; ++i) bias[i] = T::to_f32(p.bias[n0 + row + i]);
            }
#pragma unroll
            for (int tb = 0; tb < 4; ++tb) {
                u32x2 o;
                o[0] = T::from_f32(p.alpha * acc[pr][tb][4 * g] + bias[0]) | (T::from_f32(p.alpha * acc[pr][tb][4 * g + 1] + bias[1]) << 16);
                o[1] = T::from_f32(p.alpha * acc[pr][tb][4 * g + 2] + bias[2]) | (T::from_f32(p.alpha * acc[pr][tb][4 * g + 3] + bias[3]) << 16);
                *reinterpret_cast<u32x2 *>(buf + (tb * 32 + c32) * kP8OutPitch + row * 2) = o;
            }
        }
    // lane 8 t + q: 16 bytes (8 rows) q of token t of each group of eight tokens
    const int t8 = lane >> 3, q = lane & 7;
    const bool rows_ok = n0 + q * 8 < p.N;
#pragma unroll
    for (int it = 0; it < 16; ++it) {
        const int token = it * 8 + t8;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(buf + token * kP8OutPitch + q * 16);
        if (rows_ok && tok0 + token < p.M) *reinterpret_cast<u32x4 *>(p.C + (size_t)(tok0 + token) * p.N + n0 + q * 8) = v;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// 256 x 256 panels of 16-bit weights: eight waves, both operands through LDS, fetched with loads that write LDS directly.
//
// A wave that issues v_mfma_f32_32x32x16 back to back loses matrix-core time with every other instruction it has to
// issue in between (measured: about 20 cycles per LDS read, 24 per load); with two waves per SIMD the instructions
// of one wave go out under the products of the other.  That needs both waves of a SIMD inside 256 registers each,
// so nothing is staged through registers here: a k32 slab of the panel (16 weight tiles of 16 rows x 32 k, 1 KiB
// each, as they lie in layout A; 16 chunks of 16 tokens x 32 k) is copied into LDS by 32 buffer loads with the LDS
// bit, four per wave: the weight tiles addressed by the thread id alone (the descriptor adds 16 bytes per lane, no
// address register), the token chunks with a per-lane offset (lane 4 t + j fetches octet j ^ (t / 4) of token t, so that
// four lanes cover 64 consecutive bytes of a token row and the operand reads below meet no bank twice).
// Wave w = (token half w / 4, row quarter w % 4) multiplies 64 rows x 128 tokens: per k16 step two weight operands (two
// vertically adjacent tiles read as one 32-row operand: lane 32 g + i takes row i % 16 of tile i / 16, octet g) and four
// token operands feed eight products.
//
// Ring of four slabs (128 KiB).  While slab s is multiplied, slab s + 1 is complete and published, slab s + 2 is landing
// and the loads of slab s + 3 go out into the buffer that slab s - 1 has left; one wait (this wave's loads of slab
// s + 2) and one barrier per slab publish slab s + 2 and retire slab s.  The operands of the first step of slab s + 1
// are read before that barrier, so no wave stands idle behind it.  The barrier is the bare instruction: the fence that
// comes with __syncthreads() would wait for every load in flight.
constexpr int kP8Slab = 2048;                                  // 16-byte granules of a slab: 1024 of weights, 1024 of tokens
constexpr size_t kP8RingBytes = (size_t)4 * kP8Slab * 16;

// the four loads of one wave for slab `slab` (counted from k = 0) into ring buffer `buf`
__device__ __forceinline__ void p8_issue(const uint8_t *a_panel, const uint16_t *b, const uint32_t (&a_soff)[2],
                                         const uint32_t (&b_voff)[2], int wave, int slab, int buf) {
    extern __shared__ u32x4 win[];
    __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc((void *)a_panel, 16, 0xffffffffu, 1 << 23);
    __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc((void *)b, 0, 0xffffffffu, 0x00020000);
    const int dst = buf * kP8Slab;
#pragma unroll
    for (int i = 0; i < 2; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, win + dst + (2 * wave + i) * 64, 16, 0, a_soff[i] + slab * 1024, 0, 0);
#pragma unroll
    for (int i = 0; i < 2; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, win + dst + 1024 + (2 * wave + i) * 64, 16, b_voff[i], slab * 64, 0, 0);
}

//
// Grid: without K slices the workgroup ids of an XCD walk bands of p.band groups of eight row tiles in chunks of
// p.chunk token tiles, so that the 32 workgroups an XCD runs at a time cover 8 x 4 (row tiles x token tiles) and share
// both operands through its L2; with the token tiles of two row tiles side by side (2 x 16) the same product took
// 17 % longer (8192 x 8192, 4096 tokens: 491 against 413 us).  A fifth slab of LDS (160 KiB) changed nothing.
template <class T>
__global__ void __launch_bounds__(512) gemm_panel8_kernel(PanelArgs p) {
    constexpr int RING = 4;
    extern __shared__ u32x4 win[];
    constexpr int PR = 2, TB = 4;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave & 3, wt = wave >> 2;

    // workgroup -> (row tile, k slice, token tile), as in gemm_panel_kernel
    const int xcd = blockIdx.x & 7;
    int u = blockIdx.x >> 3;
    int SK, sk, tt, rt;
    if (p.band > 0) {
        const int TT = p.token_tiles, groups8 = (p.row_tiles + 7) >> 3, RB = p.band, TC = p.chunk;
        const int band = u / (RB * TT);
        const int nb = min(RB, groups8 - band * RB);           // groups of row tiles in this band
        const int v = u - band * RB * TT;
        const int c = v / (nb * TC);
        const int tc = min(TC, TT - c * TC);                   // token tiles in this chunk
        const int w = v - c * nb * TC;
        SK = 1, sk = 0;
        tt = c * TC + w % tc;
        rt = (band * RB + w / tc) * 8 + xcd;
    } else {
        const int whole_wgs = p.whole_groups * p.token_tiles;
        const bool sliced = u >= whole_wgs;
        SK = sliced ? p.SK : 1;
        if (sliced) u -= whole_wgs;
        tt = u % p.token_tiles;
        u /= p.token_tiles;
        sk = u % SK;
        rt = ((sliced ? p.whole_groups : 0) + u / SK) * 8 + xcd;
    }
    if (rt >= p.row_tiles) return;

    const int groups = p.N >> 4;
    const int rgp = rt * 16;                                   // first row group of the panel
    const int rg0 = rgp + wr * 4;                              // of this wave
    const int tok0 = tt * 256;
    const int nwin_total = p.K / 64;                           // slices are cut in windows of 64 k, as the host counts them
    const int wbeg = (int)((long long)sk * nwin_total / SK);
    const int slab0 = 2 * wbeg;
    const int nslab = 2 * ((int)((long long)(sk + 1) * nwin_total / SK) - wbeg);

    // sources of this wave's loads: weight tiles 2 wave, 2 wave + 1 of the panel (rows past N: a copy of the last row
    // group, never stored), token chunks 2 wave, 2 wave + 1 (tokens past M: the last token)
    const uint8_t *a_panel = p.A + (size_t)rgp * p.K * 32;
    uint32_t a_soff[2], b_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int rg = min(rgp + 2 * wave + i, groups - 1);
        a_soff[i] = (uint32_t)(rg - rgp) * (uint32_t)p.K * 32u;
        const int t = lane >> 2, oct = (lane & 3) ^ ((t >> 2) & 3);
        const int tok = min(tok0 + (2 * wave + i) * 16 + t, p.M - 1);
        b_voff[i] = (uint32_t)tok * (uint32_t)p.K * 2u + oct * 16;
    }
    // operand reads (granules inside a slab, first k16 step; the second step is + 32 for weights, ^ 2 for tokens)
    const int g = lane >> 5, i32 = lane & 31, t16 = i32 & 15, hi = i32 >> 4;
    const int a_idx = (wr * 4 + hi) * 64 + g * 16 + t16;                                         // + 128 pr
    const int b_idx = 1024 + (wt * 8 + hi) * 64 + 4 * t16 + (g ^ ((t16 >> 2) & 3));           // + 128 tb

    f32x16 acc[PR][TB];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

    u32x4 a0[PR], a1[PR], b0[TB], b1[TB];
    auto rd = [&](u32x4 (&a)[PR], u32x4 (&b)[TB], int buf, int hs) {
        const u32x4 *src = win + buf * kP8Slab;
#pragma unroll
        for (int pr = 0; pr < PR; ++pr) a[pr] = src[a_idx + 128 * pr + hs * 32];
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) b[tb] = src[(b_idx ^ (hs * 2)) + 128 * tb];
    };
    auto mm = [&](const u32x4 (&a)[PR], const u32x4 (&b)[TB]) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int pr = 0; pr < PR; ++pr) acc[pr][tb] = T::mfma32(a[pr], b[tb], acc[pr][tb]);
    };
    // slabs past the end of the slice are fetched as copies of its last slab and never multiplied, which keeps the
    // count of loads in flight the same in every trip
    const int last = slab0 + nslab - 1;
#pragma unroll
    for (int i = 0; i < RING - 1; ++i) p8_issue(a_panel, p.B, a_soff, b_voff, wave, min(slab0 + i, last), i);
    wait_vmcnt_le<4 * (RING - 3)>();                           // slabs 0 and 1 of this wave have landed
    bare_barrier();
    rd(a0, b0, 0, 0);
    int cur = 0;                                               // ring buffer of slab s
    for (int s = 0; s < nslab; ++s) {
        const int nxt = cur == RING - 1 ? 0 : cur + 1, prv = cur == 0 ? RING - 1 : cur - 1;
        p8_issue(a_panel, p.B, a_soff, b_voff, wave, min(slab0 + s + RING - 1, last), prv);
        rd(a1, b1, cur, 1);
        mm(a0, b0);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (m != 3 && m != 7) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (m < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        rd(a0, b0, nxt, 0);
        mm(a1, b1);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (m != 3 && m != 7) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt_le<4 * (RING - 3)>();                       // this wave's loads of slab s + 2 have landed
        bare_barrier();
        cur = nxt;
    }
    __builtin_amdgcn_s_waitcnt(0);                             // nothing may still be writing LDS when the ring is given up
    mfma_settle();
    __syncthreads();
    if (SK == 1) p8_store_panel<T>(p, acc, rg0, tok0 + wt * 128, wave, lane, win);
    else panel_finish<T, PR, TB, 8, 2>(p, acc, rg0, tok0 + wt * 128, SK, sk, rt, tt, wave, lane, reinterpret_cast<int *>(win));
}

// The same panel for soft-FP8 weights.  The fp8 tiles (512 bytes) land in a small ring of their own (three slabs of
// 8 KiB behind the four bf16 slabs: 152 KiB in all); every wave widens the two tiles it fetched itself, two slabs ahead of
// their use, lane by lane (8 bytes in, 16 bytes out at the same lane's place: the tile order does not change) into the
// bf16 slab, so that each weight is widened once per workgroup and the multiplying loop is the 16-bit one.  Per slab and
// wave: two token-chunk loads, one fp8 load (its two tiles, 32 lanes each), two 8-byte LDS reads, 32 conversion
// instructions, two 16-byte LDS writes, sixteen products.
constexpr int kP8RawSlab = 512;                                // granules of a slab of fp8 tiles
constexpr size_t kP8Fp8LdsBytes = (size_t)(4 * kP8Slab + 3 * kP8RawSlab) * 16;

__device__ __forceinline__ void p8_issue_fp8(const uint8_t *a_panel, const uint16_t *b, uint32_t a_voff, const uint32_t *b_voff,
                                             int wave, int slab_b, int buf_b, int slab_a, int buf_a) {
    extern __shared__ u32x4 win[];
    __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc((void *)a_panel, 0, 0xffffffffu, 0x00020000);
    __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc((void *)b, 0, 0xffffffffu, 0x00020000);
#pragma unroll
    for (int i = 0; i < 2; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, win + buf_b * kP8Slab + 1024 + (2 * wave + i) * 64, 16, b_voff[i], slab_b * 64, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, win + 4 * kP8Slab + buf_a * kP8RawSlab + 2 * wave * 32, 16, a_voff, slab_a * 512, 0, 0);
}

template <class T>
__global__ void __launch_bounds__(512) gemm_panel8_fp8_kernel(PanelArgs p) {
    extern __shared__ u32x4 win[];
    constexpr int PR = 2, TB = 4;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave & 3, wt = wave >> 2;
    const int xcd = blockIdx.x & 7;
    int u = blockIdx.x >> 3;
    int SK, sk, tt, rt;
    if (p.band > 0) {
        const int TT = p.token_tiles, groups8 = (p.row_tiles + 7) >> 3, RB = p.band, TC = p.chunk;
        const int band = u / (RB * TT);
        const int nb = min(RB, groups8 - band * RB);
        const int v = u - band * RB * TT;
        const int c = v / (nb * TC);
        const int tc = min(TC, TT - c * TC);
        const int w = v - c * nb * TC;
        SK = 1, sk = 0;
        tt = c * TC + w % tc;
        rt = (band * RB + w / tc) * 8 + xcd;
    } else {
        const int whole_wgs = p.whole_groups * p.token_tiles;
        const bool sliced = u >= whole_wgs;
        SK = sliced ? p.SK : 1;
        if (sliced) u -= whole_wgs;
        tt = u % p.token_tiles;
        u /= p.token_tiles;
        sk = u % SK;
        rt = ((sliced ? p.whole_groups : 0) + u / SK) * 8 + xcd;
    }
    if (rt >= p.row_tiles) return;

    const int groups = p.N >> 4;
    const int rgp = rt * 16;
    const int rg0 = rgp + wr * 4;
    const int tok0 = tt * 256;
    const int nwin_total = p.K / 64;
    const int wbeg = (int)((long long)sk * nwin_total / SK);
    const int slab0 = 2 * wbeg;
    const int nslab = 2 * ((int)((long long)(sk + 1) * nwin_total / SK) - wbeg);
    const int scale_cols = (p.K + 127) >> 7;

    // this wave fetches and widens the tiles of row groups rgp + 2 wave, + 1 (rows past N: the last row group)
    const uint8_t *a_panel = p.A + (size_t)rgp * p.K * 16;
    const int rga = min(rgp + 2 * wave, groups - 1), rgb = min(rgp + 2 * wave + 1, groups - 1);
    const uint32_t a_voff = (uint32_t)((lane >> 5 ? rgb : rga) - rgp) * (uint32_t)p.K * 16u + (lane & 31) * 16;
    const ScaleRow srow = load_scale_row(p.scale ? p.scale + (size_t)(rga >> 3) * scale_cols : nullptr, scale_cols, lane);
    uint32_t b_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int t = lane >> 2, oct = (lane & 3) ^ ((t >> 2) & 3);
        const int tok = min(tok0 + (2 * wave + i) * 16 + t, p.M - 1);
        b_voff[i] = (uint32_t)tok * (uint32_t)p.K * 2u + oct * 16;
    }
    const int g = lane >> 5, i32 = lane & 31, t16 = i32 & 15, hi = i32 >> 4;
    const int a_idx = (wr * 4 + hi) * 64 + g * 16 + t16;
    const int b_idx = 1024 + (wt * 8 + hi) * 64 + 4 * t16 + (g ^ ((t16 >> 2) & 3));

    f32x16 acc[PR][TB];
#pragma unroll
    for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[pr][tb][e] = 0.f;

    u32x4 a0[PR], a1[PR], b0[TB], b1[TB];
    auto rd = [&](u32x4 (&a)[PR], u32x4 (&b)[TB], int buf, int hs) {
        const u32x4 *src = win + buf * kP8Slab;
#pragma unroll
        for (int pr = 0; pr < PR; ++pr) a[pr] = src[a_idx + 128 * pr + hs * 32];
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) b[tb] = src[(b_idx ^ (hs * 2)) + 128 * tb];
    };
    auto mm = [&](const u32x4 (&a)[PR], const u32x4 (&b)[TB]) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int pr = 0; pr < PR; ++pr) acc[pr][tb] = T::mfma32(a[pr], b[tb], acc[pr][tb]);
    };
    // widen this wave's two tiles of slab `slab` (counted from k = 0) from raw buffer rb into bf16 slab buffer `buf`
    auto widen = [&](int slab, int rb, int buf) {
        const float sc = scale_at(srow, slab >> 2);
        const u32x2 *raw = reinterpret_cast<const u32x2 *>(win + 4 * kP8Slab + rb * kP8RawSlab + 2 * wave * 32);
        u32x4 *dst = win + buf * kP8Slab + 2 * wave * 64;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const u32x2 f = raw[i * 64 + lane];
            uint32_t x0, x1, x2, x3;
            fp8x4_to_bf16x4(f[0], sc, x0, x1);
            fp8x4_to_bf16x4(f[1], sc, x2, x3);
            dst[i * 64 + lane] = u32x4{x0, x1, x2, x3};
        }
    };
    // Order of this wave's loads: chunks(0) raw(0) chunks(1) raw(1) chunks(2) raw(2) | raw(3) | then per trip s: chunks(s + 3)
    // raw(s + 4).  Slabs past the end of the slice are fetched (and widened) as copies of its last slab and never multiplied.
    const int last = slab0 + nslab - 1;
#pragma unroll
    for (int i = 0; i < 3; ++i) p8_issue_fp8(a_panel, p.B, a_voff, b_voff, wave, min(slab0 + i, last), i, min(slab0 + i, last), i);
    wait_vmcnt_le<3>();                                        // chunks and tiles of slabs 0 and 1 have landed
    widen(min(slab0, last), 0, 0);
    widen(min(slab0 + 1, last), 1, 1);
    {   // raw(3) into the raw buffer that slab 0 has left
        __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc((void *)a_panel, 0, 0xffffffffu, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, win + 4 * kP8Slab + 0 * kP8RawSlab + 2 * wave * 32, 16, a_voff,
                                                 min(slab0 + 3, last) * 512, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);                        // lgkmcnt(0): the widened tiles are written
    bare_barrier();
    rd(a0, b0, 0, 0);
    int cur = 0, rcur = 0;                                     // ring buffer of slab s, raw buffer of slab s
    for (int s = 0; s < nslab; ++s) {
        const int nxt = (cur + 1) & 3, nx2 = (cur + 2) & 3, prv = (cur + 3) & 3;
        const int r1 = rcur == 2 ? 0 : rcur + 1, r2 = rcur == 0 ? 2 : rcur - 1;      // raw buffers of slabs s + 1 (= s + 4), s + 2
        p8_issue_fp8(a_panel, p.B, a_voff, b_voff, wave, min(slab0 + s + 3, last), prv, min(slab0 + s + 4, last), r1);
        // the tiles of slab s + 2: everything younger than them may still be in flight (four loads in the first trip,
        // where raw(3) went out alone; six from then on)
        if (s == 0) wait_vmcnt_le<4>();
        else wait_vmcnt_le<6>();
        // the fp8 tiles are read first, widened between the products of the first half step and written after them
        const float sc = scale_at(srow, min(slab0 + s + 2, last) >> 2);
        const u32x2 *raw = reinterpret_cast<const u32x2 *>(win + 4 * kP8Slab + r2 * kP8RawSlab + 2 * wave * 32);
        const u32x2 f0 = raw[lane], f1 = raw[64 + lane];
        rd(a1, b1, cur, 1);
        u32x4 w0, w1;
        {
            uint32_t x0, x1, x2, x3;
            fp8x4_to_bf16x4(f0[0], sc, x0, x1);
            fp8x4_to_bf16x4(f0[1], sc, x2, x3);
            w0 = u32x4{x0, x1, x2, x3};
            fp8x4_to_bf16x4(f1[0], sc, x0, x1);
            fp8x4_to_bf16x4(f1[1], sc, x2, x3);
            w1 = u32x4{x0, x1, x2, x3};
        }
        mm(a0, b0);
        {
            u32x4 *dst = win + nx2 * kP8Slab + 2 * wave * 64;
            dst[lane] = w0;
            dst[64 + lane] = w1;
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);       // the LDS reads
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#pragma unroll
        for (int m = 2; m < 8; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);   // six conversion instructions
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);       // the two LDS writes
        __builtin_amdgcn_sched_barrier(0);
        rd(a0, b0, nxt, 0);
        mm(a1, b1);
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt_le<4>();                                    // this wave's chunks of slab s + 2 have landed
        __builtin_amdgcn_s_waitcnt(0xc07f);                    // and its widened tiles are written
        bare_barrier();
        cur = nxt;
        rcur = r1;
    }
    __builtin_amdgcn_s_waitcnt(0);
    mfma_settle();
    __syncthreads();
    if (SK == 1) p8_store_panel<T>(p, acc, rg0, tok0 + wt * 128, wave, lane, win);
    else panel_finish<T, PR, TB, 8, 2>(p, acc, rg0, tok0 + wt * 128, SK, sk, rt, tt, wave, lane, reinterpret_cast<int *>(win));
}

// Tokens per panel when the caller leaves the choice open.  Workgroups run one per CU in rounds; a 256-token panel
// takes 1.3 to 1.5 times as long as a 128-token one for 16-bit weights (eight-wave kernel) and 1.84 times for soft-FP8
// ones (measured), so the width with the cheaper sum of rounds wins.
int panel_tokens(int m, int n, bool fp8) {
    const int cus = device_cus();
    const long long row_tiles = (n + kPanelRowsPerWg - 1) / kPanelRowsPerWg;
    const long long rounds128 = (row_tiles * ((m + 127) / 128) + cus - 1) / cus;
    const long long rounds256 = (row_tiles * ((m + 255) / 256) + cus - 1) / cus;
    return rounds256 * (fp8 ? 184 : 140) < rounds128 * 100 ? 256 : 128;
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
    PanelArgs p = {};
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
    if (width != 128 && width != 256) width = panel_tokens(m, n, a_kind == MLK_FP8_E4M3);
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
        // eight waves, operands through LDS
#define MLK_PANEL8(KERNEL, LDS)                                                                                        \
    do {                                                                                                           \
        static bool ready_on[64] = {};                                                                             \
        bool &ready = ready_on[dev & 63];                                                                          \
        if (!ready) {                                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&KERNEL),                            \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)(LDS));           \
            if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));                                \
            ready = true;                                                                                          \
        }                                                                                                          \
        KERNEL<<<grid, 512, LDS, s>>>(p);                                                                          \
    } while (0)
        const bool whole = p.SK == 1 && p.whole_groups == 0;
        p.band = whole ? 8 : 0;
        p.chunk = 4;
        // LDS: the ring, or the turn-around buffer of the output if that is larger
        constexpr size_t lds16 = kP8RingBytes > kP8OutBytes ? kP8RingBytes : kP8OutBytes;
        constexpr size_t lds8 = kP8Fp8LdsBytes > kP8OutBytes ? kP8Fp8LdsBytes : kP8OutBytes;
        if (a_kind == MLK_FP8_E4M3) MLK_PANEL8(gemm_panel8_fp8_kernel<BF16>, lds8);
        else if (a_kind == MLK_F16) MLK_PANEL8(gemm_panel8_kernel<F16>, lds16);
        else MLK_PANEL8(gemm_panel8_kernel<BF16>, lds16);
#undef MLK_PANEL8
    } else if (rows == 256 && a_kind == MLK_FP8_E4M3 && (p.SK == 1 || p.whole_groups > 0)) {
        // soft-FP8, panels computed whole (or only the last round's sliced): the loop that prefetches through LDS, two
        // workgroups per CU (28672 x 8192 at 1024 tokens: 616 -> 474 us); fully sliced grids and 16-bit weights stay on
        // the register-ring loop, which is ahead there
#define MLK_PANEL_LDS(TT, F8, RING)                                                                                    \
    do {                                                                                                           \
        constexpr size_t lds = PanelLdsShape<F8, 4, RING>::lds_bytes;                                              \
        static bool ready_on[64] = {};                                                                             \
        bool &ready = ready_on[dev & 63];                                                                          \
        if (!ready) {                                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_panel_lds_kernel<TT, F8, RING>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);             \
            if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));                                \
            ready = true;                                                                                          \
        }                                                                                                          \
        gemm_panel_lds_kernel<TT, F8, RING><<<grid, 256, lds, s>>>(p);                                             \
    } while (0)
        MLK_PANEL_LDS(BF16, true, 4);
#undef MLK_PANEL_LDS
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
