// Narrow GeMM (1 <= M <= 64 per weight pass) over layout-A weights with
// v_mfma_f32_16x16x32: C[M, N] = alpha * B[M, K] . A^T + bias.
//
// Work decomposition.  A workgroup owns R consecutive row groups (16 R weight
// rows) and one of SK slices of K.  Its WK waves take the slice's 32-wide k
// tiles round-robin.  For every k tile a wave loads R weight fragments (1 KiB
// each, 16 bytes per lane, coalesced, non-temporal) and CB activation
// fragments (CB = ceil(M/16) <= 4) and issues R*CB MFMAs, so each activation
// fragment is reused R times and each weight fragment CB times; weights are
// read from HBM exactly once.  Fragments are prefetched U tiles ahead in a
// register ring.  Wave partials are folded through LDS in wave order; with
// SK > 1 workgroup partials go to an fp32 workspace and the last workgroup to
// arrive for a row tile folds them in slice order, so results are
// deterministic and never depend on atomics in the data path.
//
// The same kernel serves the three operand placements of the reference:
// row-major or layout-B activations, row-major or layout-C output.  Because
// the accumulation order is identical, layout-C output followed by the
// layout-C -> row-major permutation equals the row-major output bit for bit.
//
// (template code shared by the per-type translation units mlk_gemm_f16.hip, mlk_gemm_bf16.hip and
// mlk_gemm_fp8.hip, which instantiate launch_modes<> so that they compile in parallel)
//
// Algorithmic traffic per call: N*K*sizeof(W) (+ scales) + M*K*2 + M*N*2 bytes.
#pragma once

#include "mlk_tile.cuh"

namespace mlk {



struct GemmArgs {
    const uint8_t *A;
    const uint16_t *B;
    uint16_t *C;
    const uint16_t *bias;
    const float *scale;
    float *partial;      // [SK][row_tiles][R*CB][64] x 4 floats
    int *counters;       // [row_tiles], zero between calls
    int M;               // tokens handled by this launch (columns cb0*16 .. )
    int M_total;         // tokens in the whole problem (row count of B / C)
    int cb0;             // first 16-token block of this launch
    int N, K;
    int WK, SK;
    int depth;           // 0 = default ring depth, else 2, 4, 6 or 8 (used when one token block is in flight)
    int rotate;
    float alpha;
};

// Granules (16 bytes) between the activation fragments of neighbouring k tiles in a staged window.
__host__ __device__ constexpr int stage_win_stride(int cb) { return cb * 68 + (cb % 2 == 0 ? 4 : 0); }

// Threads per workgroup the wave kernel is compiled for: deep register rings (many tiles x many
// k tiles in flight) get the register budget of a 256-thread workgroup instead of spilling.
__host__ __device__ constexpr int wave_kernel_threads(int ntile, int depth, bool staged) {
    return (!staged && ntile * depth >= 24 && max_threads_for_tiles(ntile) > 256) ? 256 : max_threads_for_tiles(ntile);
}

// The body of the wave kernel for the R row groups from rg0 (row tile rt of `row_tiles`, K slice sk).
// red: [WK][R*CB][64] f32x4 of LDS; the staged variant first uses it for two activation windows.
template <class T, bool FP8, int CB, int R, int BMODE, int CMODE, int U, bool STAGE, bool TWOSC = false>
__device__ __forceinline__ void gemm_wave_body(const GemmArgs &p, const int rt, const int sk, const int rg0,
                                               const int row_tiles, f32x4 *red, int &s_last) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, kept scalar
    const int q = lane >> 4, r16 = lane & 15;
    const int tiles_total = p.K >> 5;
    const int tiles_per = (tiles_total + p.SK - 1) / p.SK;
    const int tbeg = sk * tiles_per;
    const int tend = min(tiles_total, tbeg + tiles_per);
    const int mb_total = (p.M_total + 15) >> 4;
    const int scale_cols = (p.K + 127) >> 7;
    constexpr int WBYTES = FP8 ? 1 : 2;

    const uint8_t *abase[R];
#pragma unroll
    for (int r = 0; r < R; ++r) abase[r] = p.A + (size_t)(rg0 + r) * p.K * 16 * WBYTES;

    // activation fragment source for this lane
    // Lanes whose token does not exist read the last real token instead: column c of the
    // product depends only on column c of the activations, and those columns are never stored.
    const uint16_t *bptr[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        if (BMODE == MLK_B_NATIVE) {
            bptr[cb] = p.B + ((size_t)(p.cb0 + cb) * 64 + lane) * 8;
        } else {
            int tok = min((p.cb0 + cb) * 16 + r16, p.M_total - 1);
            bptr[cb] = p.B + (size_t)tok * p.K + q * 8;
        }
    }
    const size_t bstep = (BMODE == MLK_B_NATIVE) ? (size_t)mb_total * 512 : 32;  // elements per k tile

    // The R row groups of a wave share one row of block scales (R divides 8, rg0 is a multiple of R).  TWOSC: rg0
    // is arbitrary and R <= 8, so the row groups may lie in two neighbouring 128-row blocks: the first `split` of
    // them take the scales of the first block, the others those of the second.
    ScaleRow srow, srow2;
    int split = R;
    if (FP8) srow = load_scale_row(p.scale ? p.scale + (size_t)(rg0 >> 3) * scale_cols : nullptr, scale_cols, lane);
    if (FP8 && TWOSC) {
        split = 8 - (rg0 & 7);
        srow2 = load_scale_row(p.scale ? p.scale + (size_t)((rg0 + R - 1) >> 3) * scale_cols : nullptr, scale_cols, lane);
    }

    f32x4 acc[R][CB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nt = (tbeg + wave < tend) ? (tend - tbeg - wave + p.WK - 1) / p.WK : 0;

    WeightFrag<FP8> wf[U][R];
    u32x4 bf[U][CB];
    float sc[U];        // one block scale per k tile: the R row groups of a wave share a 128-row block
    float sc2[U];       // TWOSC: the scale of the second block
    auto issue = [&](int slot, int kt) {
#pragma unroll
        for (int r = 0; r < R; ++r) wf[slot][r] = load_weight_frag<FP8>(abase[r], kt, lane);
        if (FP8) sc[slot] = scale_at(srow, kt >> 2);
        if (FP8 && TWOSC) sc2[slot] = scale_at(srow2, kt >> 2);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) bf[slot][cb] = ld_global_u32x4(bptr[cb] + (size_t)kt * bstep);
    };
    auto consume = [&](int slot) {
        u32x4 a[R], b[CB];
        float sv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) sv[r] = FP8 ? ((TWOSC && r >= split) ? sc2[slot] : sc[slot]) : 1.f;
        weight_operands<FP8, R>(a, wf[slot], sv);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) b[cb] = bf[slot][cb];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[r][cb] = T::mfma(a[r], b[cb], acc[r][cb]);
    };
    if constexpr (STAGE) {
        // Row-major activations, staged: in step j the WK waves work on the window of WK
        // consecutive k tiles [tbeg + w*WK, +WK).  The workgroup fetches the window's
        // activations with row-contiguous 16-byte loads (WK*64 bytes per token), one step
        // ahead, and leaves them in LDS in MFMA fragment order (two buffers, one barrier per
        // step); each wave then reads its own tile's fragments with ds_read_b128.  Fragment
        // rows are padded (68 granules per tile, 17 per k-octet) against bank conflicts, and the fragments of
        // neighbouring k tiles start 4 modulo 8 granules apart (stage_win_stride): a staging store puts the pieces
        // of two neighbouring k tiles of one token row side by side in a group of eight lanes, and the banks
        // repeat every 8 granules.
        u32x4 *win = reinterpret_cast<u32x4 *>(red);
        constexpr int WS = stage_win_stride(CB);
        const int win_granules = p.WK * WS;
        const int nwin = (tend - tbeg) / p.WK;            // exact: the host only stages when WK divides the slice
        const int cols = p.WK * 4;                        // 16-byte granules per token in a window
        const int sh = __builtin_ctz(cols);
        int rot = (nwin > 0 && p.rotate) ? (int)(((unsigned)rt * 2654435761u >> 7) % (unsigned)nwin) : 0;
        int w_stage = rot, w_issue = rot;
        auto advance = [&](int &w) {
            int cur = w;
            w = (w + 1 == nwin) ? 0 : w + 1;
            return cur;
        };
        u32x4 breg[CB];
        auto stage_load = [&]() {
            const int tile0 = tbeg + advance(w_stage) * p.WK;
#pragma unroll
            for (int i = 0; i < CB; ++i) {
                const int g = threadIdx.x + i * blockDim.x;
                if constexpr (BMODE == MLK_B_NATIVE) {
                    // layout-B: the fragment of (k tile, token block) is 1 KiB in one piece, already in MFMA order
                    const int f = g >> 6, w = f / CB, cb = f - w * CB;
                    breg[i] = ld_global_u32x4(p.B + (((size_t)(tile0 + w) * mb_total + p.cb0 + cb) * 64 + (g & 63)) * 8);
                } else {
                    const int row = g >> sh, colg = g & (cols - 1);
                    const int tok = min(p.cb0 * 16 + row, p.M_total - 1);
                    breg[i] = ld_global_u32x4(p.B + (size_t)tok * p.K + (size_t)tile0 * 32 + colg * 8);
                }
            }
        };
        auto stage_store = [&](int buf) {
#pragma unroll
            for (int i = 0; i < CB; ++i) {
                const int g = threadIdx.x + i * blockDim.x;
                if constexpr (BMODE == MLK_B_NATIVE) {
                    const int f = g >> 6, w = f / CB, cb = f - w * CB, j = g & 63;
                    win[buf * win_granules + w * WS + cb * 68 + (j >> 4) * 17 + (j & 15)] = breg[i];
                } else {
                    const int row = g >> sh, colg = g & (cols - 1);
                    win[buf * win_granules + (colg >> 2) * WS + (row >> 4) * 68 + (colg & 3) * 17 + (row & 15)] = breg[i];
                }
            }
        };
        auto issue_a = [&](int slot) {
            const int kt = tbeg + advance(w_issue) * p.WK + wave;
#pragma unroll
            for (int r = 0; r < R; ++r) wf[slot][r] = load_weight_frag<FP8>(abase[r], kt, lane);
            if (FP8) sc[slot] = scale_at(srow, kt >> 2);
            if (FP8 && TWOSC) sc2[slot] = scale_at(srow2, kt >> 2);
        };
        auto step = [&](int slot, int buf, bool do_stage, bool do_issue) {
            // pinned ahead of the products: the compiler would sink these loads to the parking stores below
            if (do_stage) stage_load();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) bf[slot][cb] = win[buf * win_granules + wave * WS + cb * 68 + q * 17 + r16];
            consume(slot);
            if (do_issue) issue_a(slot);
            __builtin_amdgcn_sched_barrier(0);
            if (do_stage) stage_store(buf ^ 1);
            __syncthreads();
        };
        // (Loads return in order, so the wait before the parking stores is also the wait for the weights requested
        // at the end of the previous step: two slots behave like one window in flight across the barrier.  Three
        // slots with the activations requested ahead of the youngest weights, so that two windows stay in flight,
        // measured 10 % slower at 40 to 64 tokens: more requests in flight per CU do not raise its bandwidth.)
        static_assert(U % 2 == 0, "the staged loop alternates two LDS buffers inside a U-step unroll");
        if (nwin > 0) {
            stage_load();
            stage_store(0);
            int j = 0;
            if (nwin >= 2 * U) {
                // Lead-in of the unrolled loop: all U windows requested without conditions and the first one
                // waited for, which is the state every trip of the loop leaves behind (U - 1 windows in flight,
                // the current one landed).  Entered in any other state the loop would be compiled to wait for
                // all of its loads at the top of every trip.
#pragma unroll
                for (int u = 0; u < U; ++u) issue_a(u);
                asm volatile("" ::"v"(wf[0][R - 1].v));
                __syncthreads();
                for (; j + 2 * U <= nwin; j += U) {
#pragma unroll
                    for (int u = 0; u < U; ++u) step(u, u & 1, true, true);
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (u < nwin) issue_a(u);
                __syncthreads();
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (j + u < nwin) step(u, u & 1, j + u + 1 < nwin, j + u + U < nwin);
            j += U;
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (j + u < nwin) step(u, u & 1, j + u + 1 < nwin, false);
        }
        __syncthreads();   // the windows are dead; the same LDS now serves the wave fold
    } else {
        // The wave visits its k tiles in a rotated order that differs from row tile to row tile:
        // workgroups that run side by side then read different parts of the (small, shared)
        // activation matrix at any moment instead of all hitting the same cache lines.
        int jcur = (nt > 0 && p.rotate) ? (int)(((unsigned)rt * 2654435761u >> 7) % (unsigned)nt) : 0;
        auto next_tile = [&]() {
            int t = tbeg + wave + jcur * p.WK;
            jcur = (jcur + 1 == nt) ? 0 : jcur + 1;
            return t;
        };

        // Register ring of U k-tiles; the steady-state loop is branch-free so the loads stay
        // U tiles deep in flight.
        if (nt >= U) {
    #pragma unroll
            for (int u = 0; u < U; ++u) issue(u, next_tile());
            int i = 0;
            for (; i + 2 * U <= nt; i += U) {
    #pragma unroll
                for (int u = 0; u < U; ++u) {
                    consume(u);
                    issue(u, next_tile());
                    __builtin_amdgcn_sched_barrier(0);  // keep each refill right behind its consume
                }
            }
            const int rem = nt - i - U;
    #pragma unroll
            for (int u = 0; u < U; ++u) {
                consume(u);
                if (u < rem) issue(u, next_tile());
            }
    #pragma unroll
            for (int u = 0; u < U; ++u)
                if (u < rem) consume(u);
        } else {
    #pragma unroll
            for (int u = 0; u < U; ++u)
                if (u < nt) issue(u, next_tile());
    #pragma unroll
            for (int u = 0; u < U; ++u)
                if (u < nt) consume(u);
        }

    }
    mfma_settle();

    constexpr int NTILE = R * CB;

    auto epilogue = [&](int j, f32x4 v) {
        const int r = j / CB, cb = j - r * CB;
        const int n = (rg0 + r) * 16 + 4 * q;
        const int tok = (p.cb0 + cb) * 16 + r16;
        if (tok >= p.M_total) return;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[i] = p.alpha * v[i];
            if (p.bias) o[i] += T::to_f32(p.bias[n + i]);
        }
        size_t off;
        if (CMODE == MLK_C_NATIVE)
            off = ((((size_t)(n >> 5) * mb_total + (tok >> 4)) * 4 + ((n & 31) >> 3)) * 16 + (tok & 15)) * 8 + (n & 7);
        else
            off = (size_t)tok * p.N + n;
        store4<T>(p.C + off, o[0], o[1], o[2], o[3]);
    };
    f32x4 *part = reinterpret_cast<f32x4 *>(p.partial);
    // 64-lane group of accumulator tile j in slice s (two planes of 8-byte halves, see st_agent_planar)
    auto group_at = [&](int s, int j) -> f32x4 * { return part + (((size_t)s * row_tiles + rt) * NTILE + j) * 64; };

    if (p.WK == 1) {
        // a single wave: tiles stay in registers
        if (p.SK == 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) epilogue(r * CB + cb, acc[r][cb]);
            return;
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) st_agent_planar(group_at(sk, r * CB + cb), 64, lane, acc[r][cb]);
    } else {
        // fold the WK waves through LDS in wave order; wave w then owns tiles j = w, w + WK, ...
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) red[(wave * NTILE + r * CB + cb) * 64 + lane] = acc[r][cb];
        __syncthreads();
        for (int j = wave; j < NTILE; j += p.WK) {
            f32x4 v = red[j * 64 + lane];
            for (int w = 1; w < p.WK; ++w) v += red[(w * NTILE + j) * 64 + lane];
            if (p.SK == 1) epilogue(j, v);
            else st_agent_planar(group_at(sk, j), 64, lane, v);
        }
        if (p.SK == 1) return;
    }

    // ---- K split across workgroups: the partial is published with agent-coherent stores, the
    // last workgroup to arrive for this row tile folds all slices in slice order.  Every wave
    // waits for its own stores to be acknowledged before the barrier; the arrival counter is
    // bumped after the barrier, so a workgroup that sees SK-1 earlier arrivals can read all
    // partials.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        int prev = __hip_atomic_fetch_add(&p.counters[rt], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == p.SK - 1);
        if (s_last) __hip_atomic_store(&p.counters[rt], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    for (int j = wave; j < NTILE; j += p.WK) {
        epilogue(j, fold_agent_planar([&](int s) { return group_at(s, j); }, p.SK, 64, lane));
    }
}

template <class T, bool FP8, int CB, int R, int BMODE, int CMODE, int U, bool STAGE>
__global__ void __launch_bounds__(wave_kernel_threads(R *CB, U, STAGE)) gemm_wave_kernel(GemmArgs p) {
    extern __shared__ f32x4 red[];
    __shared__ int s_last;
    const int rt = blockIdx.x / p.SK;
    gemm_wave_body<T, FP8, CB, R, BMODE, CMODE, U, STAGE>(p, rt, blockIdx.x % p.SK, rt * R, gridDim.x / p.SK, red, s_last);
}

// Kernel id 4: one workgroup per CU, the row groups dealt out as evenly as possible, so a workgroup
// owns floor or ceil(groups / grid) consecutive row groups: RMAX or RMAX - 1.  Both cases run the
// fully unrolled body; the test is uniform for the workgroup.  Row-major operands, no K split.  STAGE: the
// activations of a window of WK k tiles are fetched once per workgroup and shared by all its row groups through
// LDS (three and four token blocks).
template <class T, int CB, int RMAX, int U, bool STAGE = false, bool FP8 = false, int BMODE = MLK_B_ROWMAJOR,
          int CMODE = MLK_C_ROWMAJOR>
__global__ void __launch_bounds__(STAGE ? 512 : wave_kernel_threads(RMAX *CB, U, STAGE)) gemm_wave_balanced_kernel(GemmArgs p) {
    extern __shared__ f32x4 red[];
    __shared__ int s_last;
    const int groups = p.N >> 4;
    const int rt = blockIdx.x;
    const int rg0 = (int)((long long)rt * groups / (int)gridDim.x);
    const int nr = (int)((long long)(rt + 1) * groups / (int)gridDim.x) - rg0;
    // soft-FP8: a workgroup's row groups start anywhere, so they may straddle two 128-row blocks of scales
    if (nr == RMAX)
        gemm_wave_body<T, FP8, CB, RMAX, BMODE, CMODE, U, STAGE, FP8>(p, rt, 0, rg0, gridDim.x, red, s_last);
    else
        gemm_wave_body<T, FP8, CB, RMAX - 1, BMODE, CMODE, U, STAGE, FP8>(p, rt, 0, rg0, gridDim.x, red, s_last);
}

// Kernel 2: row-shared tile kernel (see mlk_tile.cuh).  Four waves per workgroup, R row groups
// per wave, activations of every k window staged once per workgroup in LDS; K is split across
// workgroups only (SK), folded by the last workgroup to arrive with agent-coherent loads.
template <class T, bool FP8, int CB, int R, int BMODE, int CMODE>
__global__ void __launch_bounds__(256) gemm_tile_kernel(GemmArgs p) {
    extern __shared__ u32x4 tile_win[];
    __shared__ int s_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4, r16 = lane & 15;
    const int sk = blockIdx.x % p.SK;
    const int rt = blockIdx.x / p.SK;
    const int rg0 = (rt * kTileWaves + wave) * R;
    const int tiles_total = p.K >> 5;
    const int tiles_per = tiles_total / p.SK;          // host: a whole number of windows
    const int tbeg = sk * tiles_per, tend = tbeg + tiles_per;
    const int mb_total = (p.M_total + 15) >> 4;
    const int scale_cols = (p.K + 127) >> 7;
    constexpr int WBYTES = FP8 ? 1 : 2;

    const uint8_t *abase[R];
    ScaleRow srow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        abase[r] = p.A + (size_t)(rg0 + r) * p.K * 16 * WBYTES;
        if (FP8)
            srow[r] = load_scale_row(p.scale ? p.scale + (size_t)((rg0 + r) >> 3) * scale_cols : nullptr, scale_cols, lane);
    }
    TileBSource<CB> bs;
    bs.native_token_major = false;
    if (BMODE == MLK_B_NATIVE) {
        bs.native_tile_stride = (size_t)mb_total * 512;
        bs.row[0] = p.B + (size_t)p.cb0 * 512;
    } else {
        bs.native_tile_stride = 0;
#pragma unroll
        for (int i = 0; i < tile_granules_per_thread<CB>(); ++i) {
            int block, token, colg;
            tile_row_of<CB>(i, threadIdx.x, block, token, colg);
            const int tok = min((p.cb0 + block) * 16 + token, p.M_total - 1);
            bs.row[i] = p.B + (size_t)tok * p.K + colg * 8;
        }
    }
    f32x4 acc[R][CB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // token blocks of this launch: exactly CB, except that 5 and 7 blocks run in the 6- and 8-wide instantiations
    const int nb = CB > 4 ? (p.M + 15) >> 4 : CB;
    TileLoop<T, FP8, CB, R>::run(acc, abase, srow, bs, tbeg, tend, tile_win, p.rotate ? rt : 0, nb);

    constexpr int NTILE = R * CB;
    const int row_tiles = gridDim.x / p.SK;
    auto epilogue = [&](int r, int cb, f32x4 v) {
        if (cb >= nb) return;
        const int n = (rg0 + r) * 16 + 4 * q;
        const int tok = (p.cb0 + cb) * 16 + r16;
        if (tok >= p.M_total) return;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[i] = p.alpha * v[i];
            if (p.bias) o[i] += T::to_f32(p.bias[n + i]);
        }
        size_t off;
        if (CMODE == MLK_C_NATIVE)
            off = ((((size_t)(n >> 5) * mb_total + (tok >> 4)) * 4 + ((n & 31) >> 3)) * 16 + (tok & 15)) * 8 + (n & 7);
        else
            off = (size_t)tok * p.N + n;
        store4<T>(p.C + off, o[0], o[1], o[2], o[3]);
    };
    if (p.SK == 1) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) epilogue(r, cb, acc[r][cb]);
        return;
    }
    f32x4 *part = reinterpret_cast<f32x4 *>(p.partial);
    auto group_at = [&](int s, int j) -> f32x4 * {
        return part + ((((size_t)s * row_tiles + rt) * kTileWaves + wave) * NTILE + j) * 64;
    };
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) st_agent_planar(group_at(sk, r * CB + cb), 64, lane, acc[r][cb]);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        int prev = __hip_atomic_fetch_add(&p.counters[rt], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == p.SK - 1);
        if (s_last) __hip_atomic_store(&p.counters[rt], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            epilogue(r, cb, fold_agent_planar([&](int s) { return group_at(s, r * CB + cb); }, p.SK, 64, lane));
        }
}

// Can kernel 2 run this problem with these parameters?
static bool tile_kernel_fits(const GemmArgs &p, int R, int CB) {
    const int tiles_total = p.K / 32;
    const int kw = CB > 4 ? 2 : 4;                       // tile_kw<CB>()
    return (p.N / 16) % (kTileWaves * R) == 0 && p.SK >= 1 && tiles_total % (p.SK * kw) == 0;
}

template <class T, bool FP8, int CB, int R, int BMODE, int CMODE>
static int launch_tile(const GemmArgs &p, hipStream_t s) {
    int row_tiles = (p.N / 16) / (kTileWaves * R);
    gemm_tile_kernel<T, FP8, CB, R, BMODE, CMODE><<<row_tiles * p.SK, 256, tile_lds_bytes<CB>(), s>>>(p);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

template <class T, bool FP8, int CB, int R, int BMODE, int CMODE>
static int launch(const GemmArgs &p, hipStream_t s) {
    constexpr int U = (R * CB >= 8) ? 2 : ((R * CB >= 4) ? 3 : 4);
    GemmArgs q = p;
    while (q.WK * 64 > max_threads_for_tiles(R * CB) || (size_t)q.WK * R * CB * 1024 > 64 * 1024) q.WK >>= 1;
    auto grid_of = [](const GemmArgs &g) { return (g.N / 16) / R * g.SK; };
    int grid = grid_of(q);
    size_t lds = q.WK > 1 ? (size_t)q.WK * R * CB * 1024 : 0;
    if constexpr (BMODE == MLK_B_ROWMAJOR && CB >= 2) {
        // stage row-major activations through LDS when every K slice is a whole number of WK-tile windows
        // (measured: staging pays from three token blocks up, and at two token blocks with eight waves to share a
        // window; below that the direct gather wins).  Up to eight waves share a window; the two windows and the
        // fold may then need more than the 64 KiB a kernel gets without asking.
        GemmArgs st = p;
        while (st.WK > 8 || st.WK * 64 > max_threads_for_tiles(R * CB)) st.WK >>= 1;
        const int tiles_total = st.K / 32;
        const int tiles_per = (tiles_total + st.SK - 1) / st.SK;
        const size_t win_bytes = (size_t)2 * st.WK * stage_win_stride(CB) * 16;
        size_t lds_st = (size_t)st.WK * R * CB * 1024;
        if (win_bytes > lds_st) lds_st = win_bytes;
        if (g_tunable[1] && (CB >= 3 || st.WK >= 8) && st.WK >= 2 && tiles_total % st.SK == 0 && tiles_per % st.WK == 0 &&
            lds_st <= 150 * 1024) {
            constexpr int US = (R * CB >= 8) ? 2 : 4;
            if (lds_st > 48 * 1024) {
                static bool ready_on[64] = {};
                int dev = 0;
                if (hipGetDevice(&dev) != hipSuccess) dev = 0;
                if (!ready_on[dev & 63]) {
                    hipError_t e = hipFuncSetAttribute(
                        reinterpret_cast<const void *>(&gemm_wave_kernel<T, FP8, CB, R, BMODE, CMODE, US, true>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
                    if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));
                    ready_on[dev & 63] = true;
                }
            }
            gemm_wave_kernel<T, FP8, CB, R, BMODE, CMODE, US, true><<<grid_of(st), st.WK * 64, lds_st, s>>>(st);
            MLK_LAUNCH_CHECK();
            return MLK_OK;
        }
    }
    if constexpr (CB == 1 && BMODE == MLK_B_ROWMAJOR && CMODE == MLK_C_ROWMAJOR) {
        // kernel ids 12, 14, 16, 18: explicit depth of the register ring (k tiles in flight per wave)
#define MLK_DEPTH(UU)                                                                                   \
    if (q.depth == UU) {                                                                                \
        while (q.WK * 64 > wave_kernel_threads(R * CB, UU, false)) q.WK >>= 1;                          \
        gemm_wave_kernel<T, FP8, CB, R, BMODE, CMODE, UU, false><<<grid, q.WK * 64, lds, s>>>(q);       \
        MLK_LAUNCH_CHECK();                                                                             \
        return MLK_OK;                                                                                  \
    }
        MLK_DEPTH(2) MLK_DEPTH(4) MLK_DEPTH(6) MLK_DEPTH(8)
#undef MLK_DEPTH
    }
    gemm_wave_kernel<T, FP8, CB, R, BMODE, CMODE, U, false><<<grid, q.WK * 64, lds, s>>>(q);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

// What a CU can pull through its vector memory path bounds these kernels when the weight matrix has
// few rows: with a fixed number of row groups per workgroup the grid of N = 11008 at 16 tokens is 172
// workgroups, a third of the CUs idle and the others over their share.  Kernel id 4 runs one workgroup
// per CU instead.
template <class T, int CB, int RMAX, bool FP8 = false, int BMODE = MLK_B_ROWMAJOR, int CMODE = MLK_C_ROWMAJOR>
static int launch_balanced(const GemmArgs &p, int wgs, hipStream_t s) {
    constexpr int U = RMAX * CB <= 4 ? 4 : (RMAX * CB <= 8 ? 3 : 2);     // k tiles in flight per wave
    GemmArgs q = p;
    q.SK = 1;
    if (CB >= 3 || (CB == 2 && q.WK >= 8)) {
        // Three and four token blocks, and two token blocks when eight waves are asked for: the activations of a
        // window of WK k tiles are staged once per workgroup in LDS and shared by all its row groups (up to eight
        // waves, one k tile of the window each; the two windows and the fold take up to 128 KiB of LDS).  Eight
        // waves sharing one window beat two waves that gather their own activations at two token blocks
        // (11008 x 4096, 32 tokens: 17.4 against 19.3 us) and four waves at four token blocks (64 tokens: 20.8
        // against 22.4 us); sixteen waves lose again (18.6 us at 32 tokens), and at one token block the gather
        // wins (15.9 against 16.4 us).
        while (q.WK > 8) q.WK >>= 1;
        const int tiles_total = q.K / 32;
        while (q.WK >= 2 && tiles_total % q.WK != 0) q.WK >>= 1;
        auto lds_for = [](int wk) {
            const size_t win_bytes = (size_t)2 * wk * stage_win_stride(CB) * 16, fold_bytes = (size_t)wk * RMAX * CB * 1024;
            return win_bytes > fold_bytes ? win_bytes : fold_bytes;
        };
        // many row groups per workgroup: fewer waves, so that the fold of their partial sums still fits
        while (q.WK > 2 && lds_for(q.WK) > 150 * 1024) q.WK >>= 1;
        const size_t lds = lds_for(q.WK);
        if (q.WK < 2 || lds > 150 * 1024) return 1;      // does not apply: the caller falls back
        if constexpr (CB >= 2) {
            // more than 64 KiB of dynamic LDS has to be allowed once per kernel and device
            static bool ready_on[64] = {};
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess) dev = 0;
            if (!ready_on[dev & 63]) {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_wave_balanced_kernel<T, CB, RMAX, 2, true, FP8, BMODE, CMODE>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
                if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));
                ready_on[dev & 63] = true;
            }
            gemm_wave_balanced_kernel<T, CB, RMAX, 2, true, FP8, BMODE, CMODE><<<wgs, q.WK * 64, lds, s>>>(q);
            MLK_LAUNCH_CHECK();
            return MLK_OK;
        }
    }
    // soft-FP8 weights and layout-B activations take this kernel only with staged windows
    if constexpr (FP8 || BMODE != MLK_B_ROWMAJOR) {
        return 1;
    } else {
        while (q.WK * 64 > wave_kernel_threads(RMAX * CB, U, false) || (size_t)q.WK * RMAX * CB * 1024 > 64 * 1024) q.WK >>= 1;
        size_t lds = q.WK > 1 ? (size_t)q.WK * RMAX * CB * 1024 : 0;
        gemm_wave_balanced_kernel<T, CB, RMAX, U><<<wgs, q.WK * 64, lds, s>>>(q);
        MLK_LAUNCH_CHECK();
        return MLK_OK;
    }
}

// number of workgroups for kernel id 4 and the larger of the two row-group counts, or 0 when it does not apply
static int balanced_grid(const GemmArgs &p, int CB, int *r_max, int most = 4) {
    const int cus = device_cus();
    const int groups = p.N / 16;
    if (groups <= cus) return 0;
    const int r = (groups + cus - 1) / cus;
    if (r < 2 || r > most || CB > 4) return 0;
    *r_max = r;
    return cus;
}

template <class T, bool FP8, int BMODE, int CMODE>
static int launch_rc(const GemmArgs &p, int kernel_id, int R, int CB, hipStream_t s) {
#define MLK_CASE(RR, CC)                                                                        \
    if (R == RR && CB == CC)                                                                    \
        return (kernel_id == 2 && tile_kernel_fits(p, RR, CC)) ? launch_tile<T, FP8, CC, RR, BMODE, CMODE>(p, s) \
                                                          : launch<T, FP8, CC, RR, BMODE, CMODE>(p, s);
    if constexpr (!FP8 && BMODE == MLK_B_NATIVE) {
        // layout-B activations (row-major or layout-C output): kernel id 4 from two token blocks on, staged windows
        if (kernel_id == 4 && CB >= 2) {
            int r_max = 0;
            const int wgs = p.SK == 1 ? balanced_grid(p, CB, &r_max) : 0;
#define MLK_BALN(CC, RR)                                                                 \
    if (wgs && CB == CC && r_max == RR) {                                                \
        const int rc = launch_balanced<T, CC, RR, false, BMODE, CMODE>(p, wgs, s);       \
        if (rc <= 0) return rc;                                                          \
    }
            MLK_BALN(2, 2) MLK_BALN(2, 3) MLK_BALN(2, 4)
            MLK_BALN(3, 2) MLK_BALN(3, 3) MLK_BALN(3, 4)
            MLK_BALN(4, 2) MLK_BALN(4, 3) MLK_BALN(4, 4)
#undef MLK_BALN
        }
    }
    if constexpr (FP8 && BMODE == MLK_B_ROWMAJOR && CMODE == MLK_C_ROWMAJOR) {
        if (kernel_id == 4 && CB >= 2) {
            int r_max = 0;
            // soft-FP8 weights are half the bytes per k tile, so the activations weigh twice as much against them:
            // up to eight row groups per workgroup share one staged window (28672 rows: seven per workgroup)
            const int wgs = p.SK == 1 ? balanced_grid(p, CB, &r_max, 8) : 0;
#define MLK_BAL8(CC, RR)                                                  \
    if (wgs && CB == CC && r_max == RR) {                                 \
        const int rc = launch_balanced<T, CC, RR, true>(p, wgs, s);       \
        if (rc <= 0) return rc;                                           \
    }
            MLK_BAL8(2, 2) MLK_BAL8(2, 3) MLK_BAL8(2, 4)
            MLK_BAL8(3, 2) MLK_BAL8(3, 3) MLK_BAL8(3, 4)
            MLK_BAL8(4, 2) MLK_BAL8(4, 3) MLK_BAL8(4, 4)
            MLK_BAL8(2, 5) MLK_BAL8(2, 6) MLK_BAL8(2, 7) MLK_BAL8(2, 8)
            MLK_BAL8(3, 5) MLK_BAL8(3, 6) MLK_BAL8(3, 7) MLK_BAL8(3, 8)
            MLK_BAL8(4, 5) MLK_BAL8(4, 6) MLK_BAL8(4, 7) MLK_BAL8(4, 8)
#undef MLK_BAL8
        }
    }
    if constexpr (!FP8 && BMODE == MLK_B_ROWMAJOR && CMODE == MLK_C_ROWMAJOR) {
        if (kernel_id == 4) {
            int r_max = 0;
            const int wgs = p.SK == 1 ? balanced_grid(p, CB, &r_max) : 0;
#define MLK_BAL(CC, RR)                                              \
    if (wgs && CB == CC && r_max == RR) {                            \
        const int rc = launch_balanced<T, CC, RR>(p, wgs, s);        \
        if (rc <= 0) return rc;                                      \
    }
            MLK_BAL(1, 2) MLK_BAL(1, 3) MLK_BAL(1, 4)
            MLK_BAL(2, 2) MLK_BAL(2, 3) MLK_BAL(2, 4)
            MLK_BAL(3, 2) MLK_BAL(3, 3) MLK_BAL(3, 4)
            MLK_BAL(4, 2) MLK_BAL(4, 3) MLK_BAL(4, 4)
#undef MLK_BAL
        }
    }
    MLK_CASE(1, 1) MLK_CASE(1, 2) MLK_CASE(1, 3) MLK_CASE(1, 4)
    MLK_CASE(2, 1) MLK_CASE(2, 2) MLK_CASE(2, 3) MLK_CASE(2, 4)
    MLK_CASE(4, 1) MLK_CASE(4, 2) MLK_CASE(4, 3) MLK_CASE(4, 4)
#undef MLK_CASE
    // five to eight token blocks (up to 128 tokens per weight pass): row-shared kernel, row-major B and C
    if constexpr (BMODE == MLK_B_ROWMAJOR && CMODE == MLK_C_ROWMAJOR) {
        if (CB > 4) {
            const int rr = R >= 2 ? 2 : 1;
            if (!tile_kernel_fits(p, rr, CB)) return fail(MLK_ERR_INVALID, "gemm: wide pass does not tile this shape");
            if (CB <= 6) return rr == 2 ? launch_tile<T, FP8, 6, 2, BMODE, CMODE>(p, s) : launch_tile<T, FP8, 6, 1, BMODE, CMODE>(p, s);
            return rr == 2 ? launch_tile<T, FP8, 8, 2, BMODE, CMODE>(p, s) : launch_tile<T, FP8, 8, 1, BMODE, CMODE>(p, s);
        }
    }
    // eight row groups per wave: wave kernel only; more than one token block only with row-major B and C
    if (R == 8 && CB == 1) return launch<T, FP8, 1, 8, BMODE, CMODE>(p, s);
    if constexpr (BMODE == MLK_B_ROWMAJOR && CMODE == MLK_C_ROWMAJOR) {
        if (R == 8 && CB == 2) return launch<T, FP8, 2, 8, BMODE, CMODE>(p, s);
        if (R == 8 && CB == 3) return launch<T, FP8, 3, 8, BMODE, CMODE>(p, s);
        if (R == 8 && CB == 4) return launch<T, FP8, 4, 8, BMODE, CMODE>(p, s);
    }
    return fail(MLK_ERR_INVALID, "gemm: unsupported (row groups per wave, column blocks)");
}

template <class T, bool FP8>
int launch_modes(const GemmArgs &p, int kernel_id, int b_mode, int c_mode, int R, int CB, hipStream_t s) {
    if (b_mode == MLK_B_ROWMAJOR && c_mode == MLK_C_ROWMAJOR)
        return launch_rc<T, FP8, MLK_B_ROWMAJOR, MLK_C_ROWMAJOR>(p, kernel_id, R, CB, s);
    if (!FP8) {
        if (b_mode == MLK_B_NATIVE && c_mode == MLK_C_ROWMAJOR)
            return launch_rc<T, false, MLK_B_NATIVE, MLK_C_ROWMAJOR>(p, kernel_id, R, CB, s);
        if (b_mode == MLK_B_NATIVE && c_mode == MLK_C_NATIVE)
            return launch_rc<T, false, MLK_B_NATIVE, MLK_C_NATIVE>(p, kernel_id, R, CB, s);
    }
    return fail(MLK_ERR_INVALID, "gemm: unsupported operand placement");
}

}  // namespace mlk
