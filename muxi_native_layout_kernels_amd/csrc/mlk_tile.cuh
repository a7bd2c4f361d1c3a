// Row-shared tile main loop: the building block for more than one block of 16 tokens.
//
// A workgroup of four waves owns 4*R row groups (each wave R of them) and all four waves walk
// the same k tiles.  The activations of a window of KW = 4 k tiles (CB token blocks) are fetched
// once per workgroup with 16-byte loads, one window ahead, and parked in LDS in MFMA fragment
// order (two buffers, one barrier per window); every wave reads the same fragments with
// ds_read_b128 and multiplies them with its own weight fragments, which stream from HBM through a
// register ring two windows deep.  Compared with every wave gathering its own activations this
// divides the activation traffic from L2 by four and keeps it coalesced.
//
// LDS layout of a window: fragment (tile w, block cb) starts at granule (w*CB + cb)*68, k-octet q
// at +17 q, token r at +r (16-byte granules; the padding keeps the transposing stores off a
// single bank).
#pragma once

#include "mlk_gemm_tile.cuh"

namespace mlk {

constexpr int kTileWaves = 4;
constexpr int kTileKW = 4;  // k tiles (of 32) per window, up to four token blocks

// k tiles per window: four, or two when more than four token blocks share the window (LDS budget)
template <int CB>
__host__ __device__ constexpr int tile_kw() {
    return CB > 4 ? 2 : 4;
}
template <int CB>
__host__ __device__ constexpr int tile_window_granules() {
    return tile_kw<CB>() * CB * 68;
}
// Granules of a window moved by one thread (the window has 64*CB*KW, the workgroup 256 threads).
template <int CB>
__host__ __device__ constexpr int tile_granules_per_thread() {
    return CB * tile_kw<CB>() / 4;
}
// Row sources: which (token block, token, k granule) the i-th granule of thread `tid` is.
template <int CB>
__device__ __forceinline__ void tile_row_of(int i, int tid, int &block, int &token, int &colg) {
    constexpr int GPR = tile_kw<CB>() * 4;     // granules per token row in a window
    const int rowidx = (tid + 256 * i) / GPR;
    block = rowidx >> 4;
    token = rowidx & 15;
    colg = tid % GPR;
}
template <int CB>
__host__ __device__ constexpr size_t tile_lds_bytes() {
    return (size_t)2 * tile_window_granules<CB>() * 16;
}

// Where a thread's share of an activation window comes from.
//   row sources (row-major or gathered tokens): granule i of the thread is (block, token, colg)
//     = tile_row_of(i, tid) -> `row[i]` points at that token's row, + colg*8
//   native source (layout-B): the window is KW runs of CB KiB; granule index g = t + 256 i
template <int CB>
struct TileBSource {
    const uint16_t *row[tile_granules_per_thread<CB>()];  // native: only row[0] = base of the first block
    size_t native_tile_stride;  // native: elements between k tiles (MB_total * 512); 0 selects row sources
    bool native_token_major;    // native: granule order inside a block is [token][octet] instead of [octet][token]
};

template <class T, bool FP8, int CB, int R>
struct TileLoop {
    // acc[r][cb] += W[stream r][tiles tbeg..tend) . activations ; (tend - tbeg) % KW == 0.
    // Only the first `nb` (workgroup-uniform, 1..CB) token blocks are multiplied; the window is always
    // fetched whole.
    __device__ static __forceinline__ void run(f32x4 (&acc)[R][CB], const uint8_t *const (&abase)[R],
                                               const ScaleRow (&srow)[R], const TileBSource<CB> &bs, int tbeg,
                                               int tend, u32x4 *win, int rot_seed, int nb = CB) {
        constexpr int KW = tile_kw<CB>();
        constexpr int NG = tile_granules_per_thread<CB>();
        constexpr int WG = tile_window_granules<CB>();
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int q = lane >> 4, r16 = lane & 15;
        const int nwin = (tend - tbeg) / KW;
        if (nwin <= 0) return;
        int rot = (int)(((unsigned)rot_seed * 2654435761u >> 7) % (unsigned)nwin);
        int w_stage = rot, w_issue = rot;
        auto advance = [&](int &w) {
            int cur = w;
            w = (w + 1 == nwin) ? 0 : w + 1;
            return cur;
        };

        u32x4 breg[NG];
        auto stage_load = [&]() {
            const int tile0 = tbeg + advance(w_stage) * KW;
#pragma unroll
            for (int i = 0; i < NG; ++i) {
                if (bs.native_tile_stride) {
                    const int g = tid + 256 * i;
                    const int w = g / (64 * CB), rem = g - w * (64 * CB);
                    breg[i] = ld_global_u32x4(bs.row[0] + (size_t)(tile0 + w) * bs.native_tile_stride + (size_t)rem * 8);
                } else {
                    breg[i] = ld_global_u32x4(bs.row[i] + (size_t)tile0 * 32);
                }
            }
        };
        auto stage_store = [&](int buf) {
#pragma unroll
            for (int i = 0; i < NG; ++i) {
                int w, cb, qq, rr;
                if (bs.native_tile_stride) {
                    const int g = tid + 256 * i;
                    w = g / (64 * CB);
                    const int rem = g - w * (64 * CB);
                    cb = rem >> 6;
                    qq = bs.native_token_major ? (rem & 3) : ((rem >> 4) & 3);
                    rr = bs.native_token_major ? ((rem >> 2) & 15) : (rem & 15);
                } else {
                    int colg;
                    tile_row_of<CB>(i, tid, cb, rr, colg);
                    w = colg >> 2;
                    qq = colg & 3;
                }
                win[buf * WG + (w * CB + cb) * 68 + qq * 17 + rr] = breg[i];
            }
        };

        WeightFrag<FP8> wf[2][KW][R];
        float sc[2][KW][R];
        auto issue_a = [&](int slot) {
            const int tile0 = tbeg + advance(w_issue) * KW;
#pragma unroll
            for (int w = 0; w < KW; ++w)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    wf[slot][w][r] = load_weight_frag<FP8>(abase[r], tile0 + w, lane);
                    sc[slot][w][r] = FP8 ? scale_at(srow[r], (tile0 + w) >> 2) : 1.f;
                }
        };
        auto step = [&](int slot, bool do_stage, bool do_issue) {
            // The activation loads of the next window go out before the products of this one: left alone the
            // compiler sinks them to their first use, the parking stores below.  (Loads return in order, so the
            // wait before those stores is also the wait for the weights requested at the end of the previous
            // step.  Deeper weight rings, with the lead-in arranged so that the loop is entered in its own
            // steady state and no trip drains the queue, measured slower: a CU keeps a bounded number of requests
            // in flight, and queueing more of them does not raise it.)
            if (do_stage) stage_load();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int w = 0; w < KW; ++w) {
                // all fragment reads of the k tile go out first, then the products (the tests on nb
                // are uniform: scalar branches)
                u32x4 a[R], b[CB];
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
                    if (cb < nb) b[cb] = win[slot * WG + (w * CB + cb) * 68 + q * 17 + r16];
                weight_operands<FP8, R>(a, wf[slot][w], sc[slot][w]);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    if (cb < nb) {
#pragma unroll
                        for (int r = 0; r < R; ++r) acc[r][cb] = T::mfma(a[r], b[cb], acc[r][cb]);
                    }
                }
            }
            mfma_settle();
            if (do_issue) issue_a(slot);
            __builtin_amdgcn_sched_barrier(0);
            if (do_stage) stage_store(slot ^ 1);
            __syncthreads();
        };

        // window j lives in LDS buffer j & 1 and in weight slot j & 1
        stage_load();
        stage_store(0);
        issue_a(0);
        if (nwin > 1) issue_a(1);
        __syncthreads();
        int j = 0;
        for (; j + 4 <= nwin; j += 2) {
            step(0, true, true);
            step(1, true, true);
        }
        // 1..3 windows left; their weights up to window j+1 are already in flight
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (j + t < nwin) step(t & 1, j + t + 1 < nwin, j + t + 2 < nwin);
        }
    }
};

}  // namespace mlk
