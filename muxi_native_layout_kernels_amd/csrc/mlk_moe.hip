// Fused MoE for gfx950: router, token -> expert-block alignment and the two
// grouped GeMMs over per-expert layout-A weight slabs.
//
//   router      one wave per token: scores (softmax / sigmoid), optional
//               selection bias, grouped selection, iterative arg-max top-K with
//               ties to the lower id, optional renormalisation
//   align       one workgroup: per-expert counts, padding to 16-slot blocks,
//               prefix sum, block owners, and a stable scatter (ascending flat
//               pair index inside each expert) - deterministic, no atomics on
//               the output positions.  It also writes the task list the GeMMs
//               walk: (expert, first block, number of blocks <= CB).
//   gate/up     grid (row tile, task): streams the gate rows and the matching
//               up rows of W1[expert] once, gathers the task's tokens as MFMA
//               activation fragments, and stores T(silu(gate) * up) as MFMA
//               activation fragments (token-major inside a block) so the second
//               GeMM reads only the real tokens, 64 contiguous bytes each
//   down        grid (row tile): walks ALL tasks, streams W2[expert] rows, and
//               adds routing weight * product into an fp32 [tokens x rows] tile
//               in LDS; one rounding to T at the end.  This is the weighted
//               un-permute: no atomics, no intermediate [pairs, H] buffer, fixed
//               summation order.
//
// Algorithmic traffic per layer: active experts * 3*I*H*sizeof(W) (+ scales)
// + 2*T*H*2 + T*E*2 bytes; the SiLU intermediate (T*K*I*2 bytes, written and
// read once) stays in L2 / Infinity Cache for decode-sized T.
#include <math.h>

#include "mlk_moe_args.cuh"

namespace mlk {

constexpr int kMaxExperts = 256;
constexpr int kMaxTopK = 32;
constexpr int kMoeChunk = 256;     // tokens per expert-compute pass
static int g_moe_gemv1 = 1;        // experiment switch: GeMV-style kernels for a single token
static int g_moe_tile = 1;         // experiment switch: row-shared kernels for tasks of more than one token block
static inline bool moe_tile_path() { return g_moe_tile != 0; }
// Token blocks per task (the tokens of one expert that share a weight pass).  Sized for the load an
// expert sees under even routing plus three standard deviations, not for the worst case: a hotter
// expert simply gets a second task (a second pass over its weights), while every task of the launch
// pays staging work for the full width.  At most 8 with the row-shared kernels (4 without); 5 and 7
// round up to the next instantiated width.
static inline int moe_blocks_per_task(int tokens, int topk, int experts) {
    const double mean = (double)tokens * topk / experts;
    int expect = (int)(mean + 3.0 * sqrt(mean)) + 1;
    if (expect > tokens) expect = tokens;
    int cb = (expect + 15) / 16;
    int cap = moe_tile_path() ? 8 : 4;
    if (g_tunable[8] > 0 && g_tunable[8] < cap) cap = g_tunable[8];      // experiment switch: fewer blocks per task
    if (cb > cap) cb = cap;
    if (cb == 5) cb = 6;
    if (cb == 7) cb = 8;
    return cb;
}

// ------------------------------------------------------------------ router
// Largest value of the wave, in every lane: four rotations inside the rows of 16 lanes on the DPP
// path, then the four row results through scalar registers.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xf, 0xf, true));   // row_ror:8
    v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x124, 0xf, 0xf, true));   // row_ror:4
    v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x122, 0xf, 0xf, true));   // row_ror:2
    v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x121, 0xf, 0xf, true));   // row_ror:1
    const uint32_t a = __builtin_amdgcn_readlane((int)v, 0), b = __builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = __builtin_amdgcn_readlane((int)v, 32), d = __builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}

// unsigned keys in the order of the floats (-0 counts as +0), and back
__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t b = __float_as_uint(f);
    if ((b << 1) == 0u) b = 0u;
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float order_key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

// One round of "take the largest, ties to the lower index": the values sit in registers (index
// lane + 64 i).  Two wave reductions on the DPP path - no LDS, no barrier.  Returns the index.
template <int NE>
__device__ __forceinline__ uint32_t wave_argmax(const float (&v)[NE], int lane) {
    uint32_t bk = order_key(v[0]);
    uint32_t bi = (uint32_t)lane;
#pragma unroll
    for (int i = 1; i < NE; ++i) {
        const uint32_t k = order_key(v[i]);
        if (k > bk) { bk = k; bi = (uint32_t)(lane + 64 * i); }
    }
    const uint32_t top = wave_max_u32(bk);
    return ~wave_max_u32(~(bk == top ? bi : 0xffffffffu));   // lowest index among the holders
}

// LDS of one routing wave.
struct RouterLds {
    __align__(16) double ex[kMaxExperts];   // exp(x - max), for the index-order sum
    __align__(16) float sel[kMaxExperts];   // selection scores, for the group scores
    int keep[kMaxExperts];
    int pick_id[kMaxTopK];
    float pick_w[kMaxTopK];
};

// The lanes of one wave exchange values through LDS: the LDS unit runs a wave's accesses in program order, so
// all that is needed between a store and the loads of other lanes is that the compiler keeps that order.  (A
// workgroup barrier would do too, but this code also runs in a single wave of a larger workgroup.)
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Routing of one token by one wave; experts lane + 64 i live in register slot i of their lane (NE slots, so up
// to 64 NE experts).  On return lane a < topk holds pick a (id and weight bits, in output order; the weight is
// renormalised if asked for).
template <class T, int NE>
__device__ __forceinline__ void route_token(const uint16_t *__restrict__ row, int E, int n_groups, int topk_groups,
                                            int topk, int score_fun, const uint16_t *__restrict__ bias, int renorm,
                                            RouterLds &L, int lane, int &out_id, uint16_t &out_w) {
    constexpr float kLowest = -3.0e38f;
    auto round_T = [](float v) { return T::to_f32(T::from_f32(v)); };

    // scores: exp, the index-order sum and the division in float64, one rounding to fp32, one to T
    float xv[NE];
    float lmax = kLowest;
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int j = lane + 64 * i;
        xv[i] = j < E ? T::to_f32(row[j]) : kLowest;
        lmax = fmaxf(lmax, xv[i]);
    }
    float pv[NE], sv[NE];      // un-biased score and selection score, both rounded to T
    if (score_fun == 0) {
        const double mx = (double)order_key_value(wave_max_u32(order_key(lmax)));
        double ev[NE];
#pragma unroll
        for (int i = 0; i < NE; ++i) ev[i] = lane + 64 * i < E ? exp((double)xv[i] - mx) : 0.0;
        // The sum runs over the experts in index order, the same in every lane: the terms go through
        // LDS and come back sixteen at a time (eight 16-byte reads in flight), then add in order.
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (lane + 64 * i < E) L.ex[lane + 64 * i] = ev[i];
        wave_lds_sync();
        typedef __attribute__((ext_vector_type(2))) double f64x2;
        double s = 0.0;
        for (int j0 = 0; j0 < E; j0 += 16) {
            f64x2 r[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) r[t] = *reinterpret_cast<const f64x2 *>(&L.ex[j0 + 2 * t]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                if (j0 + 2 * t < E) s += r[t][0];
                if (j0 + 2 * t + 1 < E) s += r[t][1];
            }
        }
#pragma unroll
        for (int i = 0; i < NE; ++i) pv[i] = round_T((float)(ev[i] / s));
    } else {
#pragma unroll
        for (int i = 0; i < NE; ++i) pv[i] = round_T((float)(1.0 / (1.0 + exp(-(double)xv[i]))));
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int j = lane + 64 * i;
        sv[i] = (bias && j < E) ? round_T(pv[i] + T::to_f32(bias[j])) : pv[i];
        if (j >= E) { sv[i] = kLowest; pv[i] = 0.f; }
    }

    if (n_groups > 1) {
        // group scores: max of the group, or the T-sum of its two largest positive scores with a bias
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (lane + 64 * i < E) L.sel[lane + 64 * i] = sv[i];
        wave_lds_sync();
        const int per_group = E / n_groups;
        float gs[NE];
        int kept[NE];
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            const int g = lane + 64 * i;
            gs[i] = kLowest;
            kept[i] = 0;
            if (g < n_groups) {
                const float *seg = L.sel + g * per_group;
                float score = 0.f;
                if (!bias) {
#pragma unroll 8
                    for (int j = 0; j < per_group; ++j) score = seg[j] > score ? seg[j] : score;
                } else {
                    float a = 0.f, b = 0.f;  // largest, second largest positive
#pragma unroll 8
                    for (int j = 0; j < per_group; ++j) {
                        float v = seg[j];
                        if (v > a) { b = a; a = v; }
                        else if (v > b) b = v;
                    }
                    if (a > 0.f) score = round_T(a + score);
                    if (b > 0.f) score = round_T(b + score);
                }
                gs[i] = score;
            }
        }
        // keep the topk_groups best groups: largest score, ties to the lower group, a kept score becomes 0
        for (int t = 0; t < topk_groups; ++t) {
            const uint32_t pick = wave_argmax<NE>(gs, lane);
            if ((int)(pick & 63u) == lane) {
#pragma unroll
                for (int i = 0; i < NE; ++i)
                    if (i == (int)(pick >> 6)) { gs[i] = 0.f; kept[i] = 1; }
            }
        }
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (lane + 64 * i < n_groups) L.keep[lane + 64 * i] = kept[i];
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            const int j = lane + 64 * i;
            if (j < E && !L.keep[j / per_group]) { sv[i] = 0.f; pv[i] = 0.f; }
        }
    }

    // K rounds of arg-max over the selection scores, ties to the lower id; a picked score becomes 0
    for (int kk = 0; kk < topk; ++kk) {
        const uint32_t pick = wave_argmax<NE>(sv, lane);
        if ((int)(pick & 63u) == lane) {
            L.pick_id[kk] = (int)pick;
#pragma unroll
            for (int i = 0; i < NE; ++i)
                if (i == (int)(pick >> 6)) { L.pick_w[kk] = pv[i]; sv[i] = 0.f; }
        }
    }
    wave_lds_sync();

    // Lane a now takes pick a.  The softmax variant returns its picks ordered by expert id (stable for
    // equal ids): each lane counts the picks that go before its own and moves its pick there.
    int my_id = lane < topk ? L.pick_id[lane] : 0x7fffffff;
    float my_w = lane < topk ? L.pick_w[lane] : 0.f;
    if (score_fun == 0) {
        int before = 0;
        for (int b = 0; b < topk; ++b) {
            const int ib = __builtin_amdgcn_readlane(my_id, b);
            before += (ib < my_id || (ib == my_id && b < lane)) ? 1 : 0;
        }
        wave_lds_sync();
        if (lane < topk) {
            L.pick_id[before] = my_id;
            L.pick_w[before] = my_w;
        }
        wave_lds_sync();
        my_id = lane < topk ? L.pick_id[lane] : 0x7fffffff;
        my_w = lane < topk ? L.pick_w[lane] : 0.f;
    }
    float denom = 1.f;
    if (renorm) {
        float s = 0.f;      // fp32 sum in output order, the same in every lane
        for (int a = 0; a < topk; ++a) s += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), a));
        denom = round_T(s);
    }
    out_id = my_id;
    out_w = (uint16_t)T::from_f32(renorm ? my_w / denom : my_w);
}

// One wave per token; NE register slots per lane hold up to 64 NE experts.
template <class T, int NE>
__global__ void __launch_bounds__(64) router_kernel(const uint16_t *__restrict__ logits, int n_tokens, int E,
                                                    int n_groups, int topk_groups, int topk, int score_fun,
                                                    const uint16_t *__restrict__ bias, int renorm,
                                                    int32_t *__restrict__ ids, uint16_t *__restrict__ weights) {
    __shared__ RouterLds L;
    const int tok = blockIdx.x;
    const int lane = threadIdx.x;
    int id;
    uint16_t w;
    route_token<T, NE>(logits + (size_t)tok * E, E, n_groups, topk_groups, topk, score_fun, bias, renorm, L, lane, id, w);
    if (lane < topk) {
        ids[(size_t)tok * topk + lane] = id;
        weights[(size_t)tok * topk + lane] = w;
    }
}

// ------------------------------------------------------------------- align

__global__ void __launch_bounds__(1024) moe_align_kernel(const int32_t *__restrict__ topk_ids, int n_pairs, int E,
                                                         const int32_t *__restrict__ experts_map,
                                                         int32_t *__restrict__ sorted_ids,
                                                         int32_t *__restrict__ cumsum_out,
                                                         int32_t *__restrict__ padded_blocks,
                                                         int32_t *__restrict__ experts_ids, int max_blocks,
                                                         MoeTask *__restrict__ tasks, int32_t *__restrict__ n_tasks,
                                                         int cb_max) {
    constexpr int NW = 16;
    __shared__ int cnt[NW][kMaxExperts];   // per-wave counts, then per-wave write cursors
    __shared__ int start[kMaxExperts + 1]; // padded exclusive prefix
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int max_padded = n_pairs + E * 15;

    for (int i = tid; i < NW * kMaxExperts; i += 1024) (&cnt[0][0])[i] = 0;
    for (int i = tid; i < max_padded; i += 1024) sorted_ids[i] = n_pairs;   // sentinel everywhere
    for (int i = tid; i < max_blocks; i += 1024) experts_ids[i] = 0;
    __syncthreads();

    // each wave owns a contiguous range of 64-pair tiles
    const int n_tiles = (n_pairs + 63) >> 6;
    const int tiles_per = (n_tiles + NW - 1) / NW;
    const int t_beg = wave * tiles_per;
    const int t_end = min(n_tiles, t_beg + tiles_per);
    auto local_expert = [&](int i) -> int {
        if (i >= n_pairs) return -1;
        int e = topk_ids[i];
        if (experts_map) e = experts_map[e];
        return (e >= 0 && e < E) ? e : -1;
    };
    for (int t = t_beg; t < t_end; ++t) {
        int e = local_expert(t * 64 + lane);
        if (e >= 0) atomicAdd(&cnt[wave][e], 1);
    }
    __syncthreads();

    // totals -> padded prefix and task list, one thread per expert (E <= 256): inclusive scans of the padded
    // sizes and of the task counts through LDS, then every expert writes its own blocks and tasks
    __shared__ int scan_pad[kMaxExperts], scan_task[kMaxExperts];
    int total = 0, nb = 0, ntk = 0;
    if (tid < E) {
        for (int w = 0; w < NW; ++w) total += cnt[w][tid];
        nb = (total + 15) >> 4;
        ntk = (nb + cb_max - 1) / cb_max;
        scan_pad[tid] = nb << 4;
        scan_task[tid] = ntk;
    }
    __syncthreads();
    for (int d = 1; d < E; d <<= 1) {
        int a = 0, c = 0;
        if (tid < E && tid >= d) {
            a = scan_pad[tid - d];
            c = scan_task[tid - d];
        }
        __syncthreads();
        if (tid < E && tid >= d) {
            scan_pad[tid] += a;
            scan_task[tid] += c;
        }
        __syncthreads();
    }
    if (tid < E) {
        const int e = tid;
        const int run = scan_pad[e] - (nb << 4);        // exclusive
        start[e] = run;
        for (int b = 0; b < nb; ++b) experts_ids[(run >> 4) + b] = e;
        if (tasks) {
            int nt = scan_task[e] - ntk;
            for (int b = 0; b < nb; b += cb_max) {
                MoeTask tk;
                tk.expert = e;
                tk.block0 = (run >> 4) + b;
                tk.nblocks = min(cb_max, nb - b);
                tk.pad = 0;
                tasks[nt++] = tk;
            }
        }
        cumsum_out[e] = run + total;                    // where the reference's atomic cursor ends up
        if (e == E - 1) {
            const int end = scan_pad[e];
            start[E] = end;
            cumsum_out[E] = end;
            padded_blocks[0] = end >> 4;
            if (n_tasks) n_tasks[0] = scan_task[e];
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += 1024) {
        int run = start[e];
        for (int w = 0; w < NW; ++w) {
            int c = cnt[w][e];
            cnt[w][e] = run;
            run += c;
        }
    }
    __syncthreads();

    // stable scatter: inside a 64-pair tile, lanes with the same expert are ranked by lane id
    for (int t = t_beg; t < t_end; ++t) {
        const int i = t * 64 + lane;
        const int e = local_expert(i);
        unsigned long long todo = __ballot(e >= 0);
        int pos = -1;
        while (todo) {
            const int leader = __ffsll((long long)todo) - 1;
            const int le = __shfl(e, leader);
            const unsigned long long same = __ballot(e == le);
            if (e == le) {
                const unsigned long long below = same & ((1ull << lane) - 1ull);
                pos = cnt[wave][le] + __popcll(below);
            }
            __builtin_amdgcn_wave_barrier();
            if (lane == leader) cnt[wave][le] += __popcll(same);
            __builtin_amdgcn_wave_barrier();
            todo &= ~same;
        }
        if (pos >= 0) sorted_ids[pos] = i;
    }
}

// ------------------------------------------------------------ grouped GeMMs
// The SiLU intermediate between the two GeMMs is private to this file.  It is kept as MFMA
// activation fragments with the token index outermost inside a block:
// [k tile = n/32][token block][token 16][k octet 4][8 elements], so the four octets of one token
// are 64 contiguous bytes and a block that holds only c real tokens is read as c*64 bytes.
__device__ __forceinline__ size_t hbuf_offset(int n, int block, int token, int SB) {
    return ((((size_t)(n >> 5) * SB + block) * 16 + token) * 4 + ((n & 31) >> 3)) * 8 + (n & 7);
}


// Decode-sized batches (T*K <= 64 pairs): every workgroup rebuilds the tiny alignment itself
// from the routing table instead of waiting for a separate alignment launch.  One wave walks
// the distinct experts in order of first appearance; an expert's pairs keep ascending order and
// fill 16-slot blocks (block id = task id), padded with the sentinel n_pairs.
constexpr int kDecodePairs = 64;
struct DecodeTables {
    MoeTask tasks[kDecodePairs];
    int sorted[kDecodePairs * 16];
    int n_tasks;
};
__device__ __forceinline__ void build_decode_tables(DecodeTables &t, const int32_t *topk_ids,
                                                    const int32_t *experts_map, int n_pairs, int E, int lane) {
    int e = -1;
    if (lane < n_pairs) {
        e = topk_ids[lane];
        if (experts_map) e = experts_map[e];
        if (e < 0 || e >= E) e = -1;
    }
    unsigned long long todo = __ballot(e >= 0);
    int nt = 0;
    while (todo) {
        const int leader = __ffsll((long long)todo) - 1;
        const int le = __shfl(e, leader);
        const unsigned long long same = __ballot(e == le);
        const int cnt = __popcll(same);
        const int nb = (cnt + 15) >> 4;
        if (e == le) {
            const int rank = __popcll(same & ((1ull << lane) - 1ull));
            t.sorted[nt * 16 + rank] = lane;
        }
        if (lane < nb * 16 - cnt) t.sorted[nt * 16 + cnt + lane] = n_pairs;
        if (lane < nb) {
            MoeTask tk;
            tk.expert = le;
            tk.block0 = nt + lane;
            tk.nblocks = 1;
            tk.pad = 0;
            t.tasks[nt + lane] = tk;
        }
        nt += nb;
        todo &= ~same;
    }
    if (lane == 0) t.n_tasks = nt;
}

// gate/up projection with SiLU(gate) * up, one task per blockIdx.y
template <class T, bool FP8, int CB, int P, int U, bool INLINE>
__global__ void __launch_bounds__(max_threads_for_tiles(2 * P * CB)) moe_gate_up_kernel(MoeArgs p) {
    extern __shared__ f32x4 red[];  // [WK][2P*CB][64]
    __shared__ DecodeTables dec;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int task = blockIdx.y;
    // the down kernel that follows counts workgroup arrivals per output column
    if (blockIdx.x == 0 && blockIdx.y == 0)
        for (int i = threadIdx.x; i < p.n_counters; i += blockDim.x) p.counters[i] = 0;
    const MoeTask *tasks = p.tasks;
    const int32_t *sorted = p.sorted;
    int n_tasks;
    if (INLINE) {
        if (wave == 0) build_decode_tables(dec, p.topk_ids, p.experts_map, p.n_pairs, p.E, lane);
        __syncthreads();
        tasks = dec.tasks;
        sorted = dec.sorted;
        n_tasks = dec.n_tasks;
    } else {
        n_tasks = p.n_tasks[0];
    }
    if (task >= n_tasks) return;
    const MoeTask tk = tasks[task];
    const int q = lane >> 4, r16 = lane & 15;
    const int g0 = blockIdx.x * P;
    constexpr int WB = FP8 ? 1 : 2;
    constexpr int R = 2 * P;                       // weight streams per wave: gate, up, gate, up ...
    const int tiles_total = p.H >> 5;
    const int groups_i = p.I >> 4;
    const size_t slab = (size_t)2 * p.I * p.H * WB;
    const int scale_cols = p.H >> 7;

    const uint8_t *abase[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int rg = (r & 1) * groups_i + g0 + (r >> 1);
        abase[r] = p.W1 + (size_t)tk.expert * slab + (size_t)rg * p.H * 16 * WB;
    }
    // block scales of the gate rows and of the up rows (the P pairs of a wave share a 128-row block)
    ScaleRow srows[2];
    if (FP8) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int rg = h * groups_i + g0;
            srows[h] = load_scale_row(
                p.S1 ? p.S1 + ((size_t)tk.expert * (2 * p.I >> 7) + (rg >> 3)) * scale_cols : nullptr, scale_cols, lane);
        }
    }
    // Padding slots and blocks beyond the task read token 0: their columns of the product are
    // written to padding rows of the intermediate (or not at all) and never reach the output.
    const uint16_t *bptr[CB];
    bool real[CB];     // lanes of padding slots issue no activation loads at all
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        int id = p.n_pairs;
        if (cb < tk.nblocks) id = sorted[(tk.block0 + cb) * 16 + r16];
        real[cb] = id < p.n_pairs;
        bptr[cb] = p.X + (size_t)(real[cb] ? id / p.K : 0) * p.H + q * 8;
    }

    f32x4 acc[R][CB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nt = (wave < tiles_total) ? (tiles_total - wave + p.WK - 1) / p.WK : 0;
    WeightFrag<FP8> wf[U][R];
    u32x4 bf[U][CB];
    float sc[U][2];     // block scales of the gate rows and of the up rows
    auto issue = [&](int slot, int kt) {
#pragma unroll
        for (int r = 0; r < R; ++r) wf[slot][r] = load_weight_frag<FP8>(abase[r], kt, lane);
        if (FP8) {
            sc[slot][0] = scale_at(srows[0], kt >> 2);
            sc[slot][1] = scale_at(srows[1], kt >> 2);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
            if (real[cb]) bf[slot][cb] = ld_global_u32x4(bptr[cb] + (size_t)kt * 32);
    };
    auto consume = [&](int slot) {
        u32x4 a[R], b[CB];
        float sv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) sv[r] = FP8 ? sc[slot][r & 1] : 1.f;
        weight_operands<FP8, R>(a, wf[slot], sv);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) b[cb] = bf[slot][cb];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[r][cb] = T::mfma(a[r], b[cb], acc[r][cb]);
    };
    int jcur = 0;
    auto next_tile = [&]() { return wave + (jcur++) * p.WK; };
    if (nt >= U) {
#pragma unroll
        for (int u = 0; u < U; ++u) issue(u, next_tile());
        int i = 0;
        for (; i + 2 * U <= nt; i += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                consume(u);
                issue(u, next_tile());
                __builtin_amdgcn_sched_barrier(0);
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

    mfma_settle();
    // fold the waves in wave order, then SiLU(gate) * up and the layout-B store
    constexpr int NT = R * CB;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) red[(wave * NT + r * CB + cb) * 64 + lane] = acc[r][cb];
    __syncthreads();
    for (int j = wave; j < P * CB; j += p.WK) {
        const int pr = j / CB, cb = j - pr * CB;
        if (cb >= tk.nblocks) continue;
        const int jg = (2 * pr) * CB + cb, ju = (2 * pr + 1) * CB + cb;
        f32x4 g = red[jg * 64 + lane], u = red[ju * 64 + lane];
        for (int w = 1; w < p.WK; ++w) {
            g += red[(w * NT + jg) * 64 + lane];
            u += red[(w * NT + ju) * 64 + lane];
        }
        float h[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) h[i] = g[i] / (1.f + __expf(-g[i])) * u[i];
        const int n = (g0 + pr) * 16 + 4 * q;           // intermediate index = k of the down projection
        const size_t off = hbuf_offset(n, tk.block0 + cb, r16, p.SB);
        store4<T>(p.Hbuf + off, h[0], h[1], h[2], h[3]);
    }
}

// Down projection over all tasks, routing weights and the sum over a token's experts in LDS.
//
// The workgroup owns R row groups of the output and walks the task list in rounds.  In a round
// the WK waves are dealt out to up to WK tasks (WK / g waves per task, each taking every
// (WK/g)-th k tile of that task's expert), so the weight streams of all the round's experts are
// in flight together and the pipeline drains once per round, not once per expert.  The fold and
// the routing-weighted scatter into the fp32 output tile then run task by task in list order, so
// the summation order of a token's experts is fixed.
template <class T, bool FP8, int CB, int R, int U, bool INLINE>
__global__ void __launch_bounds__(max_threads_for_tiles(R *CB)) moe_down_kernel(MoeArgs p) {
    extern __shared__ f32x4 red[];  // [WK][R*CB][64] then the fp32 output tile [T][16R]
    __shared__ DecodeTables dec;
    __shared__ int s_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const MoeTask *tasks = p.tasks;
    const int32_t *sorted = p.sorted;
    if (INLINE && wave == 0) build_decode_tables(dec, p.topk_ids, p.experts_map, p.n_pairs, p.E, lane);
    const int q = lane >> 4, r16 = lane & 15;
    const int rg0 = blockIdx.x * R;
    constexpr int WB = FP8 ? 1 : 2;
    constexpr int NT = R * CB;
    // blockIdx.y = K slice (the host makes the slices equal)
    const int tiles_total = (p.I >> 5) / gridDim.y;
    const int tbeg = blockIdx.y * tiles_total;
    const size_t slab = (size_t)p.H * p.I * WB;
    const int scale_cols = p.I >> 7;
    float *ytile = reinterpret_cast<float *>(red + (size_t)p.WK * NT * 64);
    const int yrows = 16 * R;

    for (int i = threadIdx.x; i < p.T * yrows; i += blockDim.x) ytile[i] = 0.f;
    __syncthreads();

    int n_tasks;
    if (INLINE) {
        tasks = dec.tasks;
        sorted = dec.sorted;
        n_tasks = dec.n_tasks;
    } else {
        n_tasks = p.n_tasks[0];
    }
    for (int base = 0; base < n_tasks;) {
        const int g = min(p.WK, n_tasks - base);      // tasks of this round
        const int wpt = p.WK / g;                     // waves per task
        const int tl = wave / wpt;                    // this wave's task inside the round
        const int ks = wave - tl * wpt;               // and its k slice
        const bool busy = tl < g;
        const MoeTask tk = tasks[base + (busy ? tl : 0)];
        const int nt = (busy && ks < tiles_total) ? (tiles_total - ks + wpt - 1) / wpt : 0;

        const uint8_t *abase[R];
#pragma unroll
        for (int r = 0; r < R; ++r) abase[r] = p.W2 + (size_t)tk.expert * slab + (size_t)(rg0 + r) * p.I * 16 * WB;
        ScaleRow srow;
        if (FP8)
            srow = load_scale_row(
                p.S2 ? p.S2 + ((size_t)tk.expert * (p.H >> 7) + (rg0 >> 3)) * scale_cols : nullptr, scale_cols, lane);
        const uint16_t *bptr[CB];
        bool real[CB];     // lanes of padding slots issue no activation loads at all
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            real[cb] = busy && cb < tk.nblocks && sorted[(tk.block0 + cb) * 16 + r16] < p.n_pairs;
            bptr[cb] = p.Hbuf + ((size_t)(tk.block0 + (cb < tk.nblocks ? cb : 0)) * 64 + r16 * 4 + q) * 8;
        }
        const size_t bstep = (size_t)p.SB * 512;

        f32x4 acc[R][CB];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
        WeightFrag<FP8> wf[U][R];
        u32x4 bf[U][CB];
        float sc[U];
        auto issue = [&](int slot, int kt) {
#pragma unroll
            for (int r = 0; r < R; ++r) wf[slot][r] = load_weight_frag<FP8>(abase[r], kt, lane);
            if (FP8) sc[slot] = scale_at(srow, kt >> 2);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                if (real[cb]) bf[slot][cb] = ld_global_u32x4(bptr[cb] + (size_t)kt * bstep);
        };
        auto consume = [&](int slot) {
            u32x4 a[R], b[CB];
            float sv[R];
#pragma unroll
            for (int r = 0; r < R; ++r) sv[r] = FP8 ? sc[slot] : 1.f;
            weight_operands<FP8, R>(a, wf[slot], sv);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) b[cb] = bf[slot][cb];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) acc[r][cb] = T::mfma(a[r], b[cb], acc[r][cb]);
        };
        int jcur = 0;
        auto next_tile = [&]() { return tbeg + ks + (jcur++) * wpt; };
        if (nt >= U) {
#pragma unroll
            for (int u = 0; u < U; ++u) issue(u, next_tile());
            int i = 0;
            for (; i + 2 * U <= nt; i += U) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    consume(u);
                    issue(u, next_tile());
                    __builtin_amdgcn_sched_barrier(0);
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

        mfma_settle();
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) red[(wave * NT + r * CB + cb) * 64 + lane] = acc[r][cb];
        __syncthreads();
        // fold and scatter task by task (list order), tiles of one task spread over the waves
        for (int t = 0; t < g; ++t) {
            const MoeTask ft = tasks[base + t];
            for (int j = wave; j < NT; j += p.WK) {
                const int r = j / CB, cb = j - r * CB;
                if (cb >= ft.nblocks) continue;
                const int id = sorted[(ft.block0 + cb) * 16 + r16];
                if (id >= p.n_pairs) continue;
                f32x4 v = red[((t * wpt) * NT + j) * 64 + lane];
                for (int w = 1; w < wpt; ++w) v += red[((t * wpt + w) * NT + j) * 64 + lane];
                const float wt = T::to_f32(p.wts[id]);
                float *dst = ytile + (size_t)(id / p.K) * yrows + r * 16 + 4 * q;
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[i] += wt * v[i];
            }
            __syncthreads();
        }
        base += g;
    }

    if (gridDim.y == 1) {
        for (int i = threadIdx.x; i < p.T * yrows; i += blockDim.x) {
            int tok = i / yrows, row = i - tok * yrows;
            p.Y[(size_t)tok * p.H + rg0 * 16 + row] = (uint16_t)T::from_f32(ytile[i]);
        }
        return;
    }
    // K slices: publish the fp32 tile with agent-coherent stores; the last workgroup to arrive
    // for this column folds the slices in slice order.
    const int cells = p.T * yrows / 4;              // f32x4 cells of a tile
    f32x4 *part = reinterpret_cast<f32x4 *>(p.part);
    auto tile_at = [&](int sk) { return part + ((size_t)sk * gridDim.x + blockIdx.x) * cells; };
    for (int i = threadIdx.x; i < cells; i += blockDim.x)
        st_agent_planar(tile_at(blockIdx.y), cells, i, *reinterpret_cast<const f32x4 *>(ytile + 4 * i));
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        int prev = __hip_atomic_fetch_add(&p.counters[blockIdx.x], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == (int)gridDim.y - 1);
    }
    __syncthreads();
    if (!s_last) return;
    for (int i = threadIdx.x; i < cells; i += blockDim.x) {
        const f32x4 v = fold_agent_planar(tile_at, (int)gridDim.y, cells, i);
        const int e = 4 * i, tok = e / yrows, row = e - tok * yrows;
        store4<T>(p.Y + (size_t)tok * p.H + rg0 * 16 + row, v[0], v[1], v[2], v[3]);
    }
}

// ------------------------------------------------------- single-token variants (one token)
// With one token every routed pair is a GeMV.  These two kernels stream the expert rows like the
// GeMV kernel (16-byte loads, register ring, v_dot2, no MFMA) with the activation vector in LDS,
// so nothing but weights crosses the memory system.

// One tile of weights (1 KiB: 16 rows x 32 k, or 16 rows x 64 k for fp8) times the matching
// activations in LDS.  acc[0] is the lane's row (row lane&15; for fp8 row 2*(lane&7)), acc[1] the
// second fp8 row.
template <class T, bool FP8>
__device__ __forceinline__ void gemv1_tile(const u32x4 &w, float s, const u32x4 *xs, int granule, float (&acc)[2]) {
    const u32x4 xv = xs[granule];
    if (FP8) {
        uint32_t w0[4], w1[4];
        if (scale_is_pow2(s)) {
            fp8x4_to_bf16x4_pow2(w[0], s, w0[0], w0[1]);
            fp8x4_to_bf16x4_pow2(w[1], s, w0[2], w0[3]);
            fp8x4_to_bf16x4_pow2(w[2], s, w1[0], w1[1]);
            fp8x4_to_bf16x4_pow2(w[3], s, w1[2], w1[3]);
        } else {
            fp8x4_to_bf16x4(w[0], s, w0[0], w0[1]);
            fp8x4_to_bf16x4(w[1], s, w0[2], w0[3]);
            fp8x4_to_bf16x4(w[2], s, w1[0], w1[1]);
            fp8x4_to_bf16x4(w[3], s, w1[2], w1[3]);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            acc[0] = T::dot2(w0[d], xv[d], acc[0]);
            acc[1] = T::dot2(w1[d], xv[d], acc[1]);
        }
    } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) acc[0] = T::dot2(w[d], xv[d], acc[0]);
    }
}

// The nt tiles first, first + step, ... of one row group against an activation vector in LDS
// (xs is indexed by the absolute tile).  The first weight loads are put in flight, then `stage`
// runs (the wave copies the activations of its own tiles to LDS; no other wave reads them, so no
// workgroup barrier is needed), then the rest streams; the 16 row sums end in red16[0..15].
template <class T, bool FP8, int U, class Stage>
__device__ __forceinline__ void gemv1_stream(const uint8_t *rowgroup, int first, int nt, int step, const u32x4 *xs,
                                             const ScaleRow &srow, float *red16, Stage stage) {
    constexpr int TKG = FP8 ? 8 : 4;                 // activation granules (8 elements) per tile
    const int lane = threadIdx.x & 63;
    const int oct = FP8 ? (lane >> 3) : (lane >> 4);
    const u32x4 *ap = reinterpret_cast<const u32x4 *>(rowgroup) + (size_t)first * 64 + lane;
    const int stride = step * 64;
    float acc[2] = {0.f, 0.f};
    u32x4 buf[U];
    float sc[U];
    auto issue = [&](int u, int j) {
        buf[u] = ld_stream_u32x4(ap + (size_t)j * stride);
        sc[u] = FP8 ? scale_at(srow, (first + j * step) >> 1) : 1.f;
    };
    auto consume = [&](int u, int j) { gemv1_tile<T, FP8>(buf[u], sc[u], xs, (first + j * step) * TKG + oct, acc); };
    const bool full = nt >= U;
    if (full) {
#pragma unroll
        for (int u = 0; u < U; ++u) issue(u, u);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < nt) issue(u, u);
    }
    stage();
    if (full) {
        int i = 0;
        for (; i + 2 * U <= nt; i += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                consume(u, i + u);
                issue(u, i + U + u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const int rem = nt - i - U;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            consume(u, i + u);
            if (u < rem) issue(u, i + U + u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < rem) consume(u, i + U + u);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < nt) consume(u, u);
    }
#pragma unroll
    for (int a = 0; a < (FP8 ? 2 : 1); ++a) {
        float v = acc[a];
        if (FP8) v += lane_xor(v, 8);
        v += lane_xor(v, 16);
        v += lane_xor(v, 32);
        acc[a] = v;
    }
    if (FP8) {
        if (lane < 8) {
            red16[2 * lane] = acc[0];
            red16[2 * lane + 1] = acc[1];
        }
    } else if (lane < 16) {
        red16[lane] = acc[0];
    }
}

// Copy the activation granules of the tiles first, first + step, ... (nt of them) into LDS: the
// wave's own share of the vector, so the waves of a workgroup never wait for each other.
template <int TKG>
__device__ __forceinline__ void gemv1_fill(u32x4 *dst, const u32x4 *src, int first, int nt, int step, int lane) {
    for (int i = lane; i < nt * TKG; i += 64) {
        const int idx = (first + (i / TKG) * step) * TKG + (i % TKG);
        dst[idx] = src[idx];
    }
}

struct Moe1Args {
    const uint8_t *W1, *W2;
    const float *S1, *S2;
    const uint16_t *X;        // [H]
    uint16_t *Y;              // [H]
    uint16_t *Hd;             // [K][I] intermediate
    const uint16_t *wts;      // [K]
    const int32_t *topk_ids;  // [K]
    const int32_t *experts_map;
    int K, H, I, E;
    int G, WK;                // gate/up: row groups per workgroup and waves splitting K (2*G*WK waves)
    int DW;                   // down: waves per workgroup
};

// gate/up for one token: grid (I/(16 G), K); waves = (gate, up) x G row groups x WK slices of K
template <class T, bool FP8, int U>
__global__ void __launch_bounds__(1024) moe_gate_up_gemv1_kernel(Moe1Args p) {
    extern __shared__ u32x4 xs[];          // the token's hidden vector
    __shared__ float red[16][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int e = p.topk_ids[blockIdx.y];
    if (p.experts_map) e = p.experts_map[e];
    if (e < 0 || e >= p.E) return;
    const int stream = wave / (p.G * p.WK);
    const int gl = (wave / p.WK) % p.G, ks = wave % p.WK;
    constexpr int WB = FP8 ? 1 : 2;
    constexpr int TK = FP8 ? 64 : 32;
    const int col = blockIdx.x * p.G + gl;                 // 16-column group of the intermediate
    const int rg = stream * (p.I >> 4) + col;
    const uint8_t *rowgroup = p.W1 + (size_t)e * 2 * p.I * p.H * WB + (size_t)rg * p.H * 16 * WB;
    ScaleRow srow;
    if (FP8)
        srow = load_scale_row(p.S1 ? p.S1 + ((size_t)e * (2 * p.I >> 7) + (rg >> 3)) * (p.H >> 7) : nullptr, p.H >> 7, lane);
    const int tiles = p.H / TK;
    const int count = ks < tiles ? (tiles - ks + p.WK - 1) / p.WK : 0;
    constexpr int TKG = FP8 ? 8 : 4;
    gemv1_stream<T, FP8, U>(rowgroup, ks, count, p.WK, xs, srow, red[wave], [&]() {
        // the 2 G waves that share these k tiles each write the same values
        gemv1_fill<TKG>(xs, reinterpret_cast<const u32x4 *>(p.X), ks, count, p.WK, lane);
    });
    __syncthreads();
    if (threadIdx.x < 16 * p.G) {
        const int g_local = threadIdx.x >> 4, r = threadIdx.x & 15;
        float g = 0.f, u = 0.f;
        for (int w = 0; w < p.WK; ++w) {
            g += red[g_local * p.WK + w][r];
            u += red[(p.G + g_local) * p.WK + w][r];
        }
        const float h = g / (1.f + __expf(-g)) * u;
        p.Hd[(size_t)blockIdx.y * p.I + (blockIdx.x * p.G + g_local) * 16 + r] = (uint16_t)T::from_f32(h);
    }
}

// down for one token: grid (H/16); the DW waves are dealt to the K pairs, DW/K slices of K each
template <class T, bool FP8, int U>
__global__ void __launch_bounds__(1024) moe_down_gemv1_kernel(Moe1Args p) {
    extern __shared__ u32x4 hs[];          // [K][I/8] intermediates of all pairs
    __shared__ float red[16][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int WB = FP8 ? 1 : 2;
    constexpr int TK = FP8 ? 64 : 32;
    const int wpt = p.DW / p.K;            // host: K <= DW
    const int pair = wave / wpt, ks = wave - pair * wpt;
    const int gran = p.I >> 3;
    int e = -1;
    if (pair < p.K) {
        e = p.topk_ids[pair];
        if (p.experts_map) e = p.experts_map[e];
        if (e >= p.E) e = -1;
    }
    // a wave without work (absent expert) streams zero tiles and leaves zero sums
    const int ee = e >= 0 ? e : 0;
    const uint8_t *rowgroup = p.W2 + (size_t)ee * p.H * p.I * WB + (size_t)blockIdx.x * p.I * 16 * WB;
    ScaleRow srow;
    if (FP8)
        srow = load_scale_row(p.S2 ? p.S2 + ((size_t)ee * (p.H >> 7) + (blockIdx.x >> 3)) * (p.I >> 7) : nullptr,
                              p.I >> 7, lane);
    const int tiles = p.I / TK;
    const int count = (e >= 0 && ks < tiles) ? (tiles - ks + wpt - 1) / wpt : 0;
    constexpr int TKG = FP8 ? 8 : 4;
    u32x4 *mine = hs + (size_t)(pair < p.K ? pair : 0) * gran;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(p.Hd) + (size_t)(pair < p.K ? pair : 0) * gran;
    gemv1_stream<T, FP8, U>(rowgroup, ks, count, wpt, mine, srow, red[wave],
                            [&]() { gemv1_fill<TKG>(mine, src, ks, count, wpt, lane); });
    __syncthreads();
    if (threadIdx.x < 16) {
        float y = 0.f;
        for (int k = 0; k < p.K; ++k) {          // pick order; pairs of absent experts left zeros
            float s = 0.f;
            for (int w = 0; w < wpt; ++w) s += red[k * wpt + w][threadIdx.x];
            y += T::to_f32(p.wts[k]) * s;
        }
        p.Y[blockIdx.x * 16 + threadIdx.x] = (uint16_t)T::from_f32(y);
    }
}

// ------------------------------------------------ row-shared variants (more than 16 tokens)
// For tasks of two to four token blocks the four waves of a workgroup share the activation
// windows through LDS (mlk_tile.cuh) instead of gathering them per wave.

// gate/up: each wave owns P (gate, up) pairs of row groups, grid (I/(64 P), tasks)
template <class T, bool FP8, int CB, int P>
__global__ void __launch_bounds__(256) moe_gate_up_tile_kernel(MoeArgs p) {
    extern __shared__ u32x4 tile_win[];
    const int task = blockIdx.y;
    if (task >= p.n_tasks[0]) return;
    const MoeTask tk = p.tasks[task];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4, r16 = lane & 15;
    const int g0 = (blockIdx.x * kTileWaves + wave) * P;   // first row group inside the gate (and the up) half
    constexpr int WB = FP8 ? 1 : 2;
    constexpr int R = 2 * P;                               // streams: gate, up, gate, up ...
    const int groups_i = p.I >> 4;
    const size_t slab = (size_t)2 * p.I * p.H * WB;
    const int scale_cols = p.H >> 7;

    const uint8_t *abase[R];
    ScaleRow srow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int rg = (r & 1) * groups_i + g0 + (r >> 1);
        abase[r] = p.W1 + (size_t)tk.expert * slab + (size_t)rg * p.H * 16 * WB;
        if (FP8)
            srow[r] = load_scale_row(
                p.S1 ? p.S1 + ((size_t)tk.expert * (2 * p.I >> 7) + (rg >> 3)) * scale_cols : nullptr, scale_cols, lane);
    }
    TileBSource<CB> bs;
    bs.native_tile_stride = 0;
    bs.native_token_major = false;
#pragma unroll
    for (int i = 0; i < tile_granules_per_thread<CB>(); ++i) {
        int block, token, colg;
        tile_row_of<CB>(i, threadIdx.x, block, token, colg);
        int id = p.n_pairs;
        if (block < tk.nblocks) id = p.sorted[(tk.block0 + block) * 16 + token];
        bs.row[i] = p.X + (size_t)(id < p.n_pairs ? id / p.K : 0) * p.H + colg * 8;
    }
    f32x4 acc[R][CB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    TileLoop<T, FP8, CB, R>::run(acc, abase, srow, bs, 0, p.H >> 5, tile_win, blockIdx.x + 7 * task, tk.nblocks);
#pragma unroll
    for (int pr = 0; pr < P; ++pr)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            if (cb >= tk.nblocks) continue;
            float h[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                h[i] = acc[2 * pr][cb][i] / (1.f + __expf(-acc[2 * pr][cb][i])) * acc[2 * pr + 1][cb][i];
            const int n = (g0 + pr) * 16 + 4 * q;
            const size_t off = hbuf_offset(n, tk.block0 + cb, r16, p.SB);
            store4<T>(p.Hbuf + off, h[0], h[1], h[2], h[3]);
        }
}

// down: each wave owns R row groups of the output, grid (H/(64 R), tasks, K slices); the
// routing-weighted partial products go to an fp32 buffer indexed by (pair, K slice), summed per
// token in a fixed order by moe_combine_kernel
template <class T, bool FP8, int CB, int R>
__global__ void __launch_bounds__(256) moe_down_tile_kernel(MoeArgs p, float *__restrict__ O) {
    extern __shared__ u32x4 tile_win[];
    const int task = blockIdx.y;
    if (task >= p.n_tasks[0]) return;
    const MoeTask tk = p.tasks[task];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4, r16 = lane & 15;
    const int rg0 = (blockIdx.x * kTileWaves + wave) * R;
    constexpr int WB = FP8 ? 1 : 2;
    const size_t slab = (size_t)p.H * p.I * WB;
    const int scale_cols = p.I >> 7;

    const uint8_t *abase[R];
    ScaleRow srow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        abase[r] = p.W2 + (size_t)tk.expert * slab + (size_t)(rg0 + r) * p.I * 16 * WB;
        if (FP8)
            srow[r] = load_scale_row(
                p.S2 ? p.S2 + ((size_t)tk.expert * (p.H >> 7) + ((rg0 + r) >> 3)) * scale_cols : nullptr, scale_cols, lane);
    }
    TileBSource<CB> bs;
    bs.native_tile_stride = (size_t)p.SB * 512;
    bs.row[0] = p.Hbuf + (size_t)tk.block0 * 512;          // CB consecutive blocks; those past the task are never used
    bs.native_token_major = true;
    f32x4 acc[R][CB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[r][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int tiles_per = (p.I >> 5) / gridDim.z;          // host: a whole number of windows
    TileLoop<T, FP8, CB, R>::run(acc, abase, srow, bs, blockIdx.z * tiles_per, (blockIdx.z + 1) * tiles_per, tile_win,
                                 blockIdx.x + 7 * task, tk.nblocks);
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        if (cb >= tk.nblocks) continue;
        const int id = p.sorted[(tk.block0 + cb) * 16 + r16];
        if (id >= p.n_pairs) continue;
        const float wt = T::to_f32(p.wts[id]);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            f32x4 v = acc[r][cb];
            v *= wt;
            *reinterpret_cast<f32x4 *>(O + ((size_t)id * gridDim.z + blockIdx.z) * p.H + (rg0 + r) * 16 + 4 * q) = v;
        }
    }
}

// y[t] = T(sum over the token's routed pairs, in pick order, of the weighted products)
template <class T>
__global__ void __launch_bounds__(256) moe_combine_kernel(const float *__restrict__ O, uint16_t *__restrict__ Y,
                                                          const int32_t *__restrict__ topk_ids,
                                                          const int32_t *__restrict__ experts_map, int K, int H,
                                                          int E, int SKD) {
    // grid (tokens, chunks of 1024 outputs): one f32x4 cell per thread
    const int tok = blockIdx.x;
    for (int n = (blockIdx.y * blockDim.x + threadIdx.x) * 4; n < H; n += gridDim.y * blockDim.x * 4) {
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < K; ++k) {
            int e = topk_ids[tok * K + k];
            if (experts_map) e = experts_map[e];
            if (e < 0 || e >= E) continue;
            f32x4 pair = {0.f, 0.f, 0.f, 0.f};
            for (int sk = 0; sk < SKD; ++sk)
                pair += *reinterpret_cast<const f32x4 *>(O + ((size_t)(tok * K + k) * SKD + sk) * H + n);
            sum += pair;
        }
        store4<T>(Y + (size_t)tok * H + n, sum[0], sum[1], sum[2], sum[3]);
    }
}

// ----------------------------------------------------------- host-side glue
struct MoeWorkspace {
    MoeTask *tasks;
    int32_t *n_tasks;
    int32_t *sorted, *cumsum, *padded, *experts_ids;
    uint16_t *hbuf;
    float *obuf;
    int32_t *counters;
    int sb;          // token blocks the intermediate is dimensioned for
};

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Bytes of the fp32 buffer that holds the K-sliced down projections of one pass of tc tokens (defined below the
// plan it reads).
static size_t moe_obuf_bytes(int tc, int n_experts, int topk, int hidden, int inter);

static size_t carve(uint8_t *base, int tc, int E, int K, int hidden, int inter, MoeWorkspace *ws) {
    const int n_pairs = tc * K;
    const int max_padded = n_pairs + E * 15;
    int max_blocks = (max_padded + 15) / 16;
    // the in-kernel alignment numbers blocks by task: at most one block per routed pair, kDecodePairs at most
    if (max_blocks < (n_pairs < kDecodePairs ? n_pairs : kDecodePairs)) max_blocks = n_pairs < kDecodePairs ? n_pairs : kDecodePairs;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        uint8_t *ptr = base ? base + off : nullptr;
        off = align_up(off + bytes, 256);
        return ptr;
    };
    MoeWorkspace w;
    w.tasks = (MoeTask *)take(sizeof(MoeTask) * (size_t)(max_blocks + 1));
    w.n_tasks = (int32_t *)take(sizeof(int32_t));
    w.sorted = (int32_t *)take(sizeof(int32_t) * (size_t)max_padded);
    w.cumsum = (int32_t *)take(sizeof(int32_t) * (size_t)(E + 1));
    w.padded = (int32_t *)take(sizeof(int32_t));
    w.experts_ids = (int32_t *)take(sizeof(int32_t) * (size_t)max_blocks);
    // seven spare blocks: the row-shared down kernel always fetches CB <= 8 consecutive blocks
    w.sb = max_blocks + 7;
    w.hbuf = (uint16_t *)take((size_t)inter * w.sb * 16 * 2);
    // fp32 buffer of the K-sliced down projections, sized for the slices the plan of this pass really uses
    w.obuf = (float *)take(moe_obuf_bytes(tc, E, K, hidden, inter));
    w.counters = (int32_t *)take(sizeof(int32_t) * (size_t)(hidden / 16));
    if (ws) *ws = w;
    return off;
}

// Waves and dynamic LDS of the decode down kernel for R row groups per wave and CB token blocks per task:
// [WK][R*CB] accumulator tiles for the wave fold plus the fp32 output tile [T][16 R], next to the kernel's
// static tables, inside the 64 KiB a workgroup gets without a per-kernel attribute.  False when even a single
// wave does not fit (R = 4 with more than 224 tokens).
static bool moe_down_shape(int T, int R, int CB, int *wk, size_t *lds) {
    auto need = [&](int w) { return (size_t)w * R * CB * 1024 + (size_t)T * 16 * R * 4; };
    const size_t budget = 64 * 1024 - sizeof(DecodeTables) - 64;
    int w = 16;
    while (w > 1 && (w * 64 > max_threads_for_tiles(R * CB) || need(w) > budget)) w >>= 1;
    *wk = w;
    *lds = need(w);
    return need(w) <= budget;
}

// Row groups per wave (= K slices across workgroups) of the decode down kernel with one token block per
// task.  More row groups cut the re-reads of the intermediate, but the output tile grows with them: the
// preferred count is halved until the tile fits with at least four waves left to stream weights.
static int moe_down_rows(int T, int H, int I, bool fp8) {
    int r = g_tunable[7] ? g_tunable[7] : (fp8 ? 4 : 1);
    if (r != 1 && r != 2 && r != 4) r = 1;
    for (; r > 1; r >>= 1) {
        int wk;
        size_t lds;
        if ((H / 16) % r == 0 && (I / 32) % r == 0 && moe_down_shape(T, r, 1, &wk, &lds) && wk >= 4) break;
    }
    return r;
}

template <class T, bool FP8, int CB, int R, bool INLINE>
static int launch_moe_down(const MoeArgs &a, int skd, hipStream_t s) {
    constexpr int U2F = (R * CB >= 4) ? 4 : (R * CB == 1 ? 10 : 6);   // fp8 tiles are half as many bytes
    constexpr int U2 = FP8 && CB == 1 ? U2F : ((R * CB >= 4) ? 3 : (R * CB == 1 ? 8 : 4));
    MoeArgs d = a;
    size_t lds2;
    if (!moe_down_shape(a.T, R, CB, &d.WK, &lds2))
        return fail(MLK_ERR_INVALID, "moe: the down projection's output tile does not fit the workgroup's LDS");
    moe_down_kernel<T, FP8, CB, R, U2, INLINE><<<dim3(a.H / 16 / R, skd), d.WK * 64, lds2, s>>>(d);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

template <class T, bool FP8, int CB, bool INLINE>
static int launch_moe(const MoeArgs &a, int max_tasks, hipStream_t s) {
    // gate/up: one (gate, up) pair of row groups per wave for CB >= 2, two pairs for CB == 1
    constexpr int P = (CB == 1) ? 2 : 1;
    constexpr int U1 = (2 * P * CB >= 8) ? 2 : 3;
    MoeArgs g = a;
    const int groups_i = a.I / 16;
    g.WK = 4;
    while (g.WK * 64 > max_threads_for_tiles(2 * P * CB)) g.WK >>= 1;
    const int grid_x = groups_i / P;   // I % 128 == 0 so this is exact for P <= 8
    size_t lds1 = (size_t)g.WK * 2 * P * CB * 1024;
    moe_gate_up_kernel<T, FP8, CB, P, U1, INLINE><<<dim3(grid_x, max_tasks), g.WK * 64, lds1, s>>>(g);
    MLK_LAUNCH_CHECK();

    if constexpr (CB == 1) {
        // One token block: R row groups per wave cut the re-reads of the intermediate R-fold; K is
        // sliced R ways so that the grid still has a workgroup per 16 output rows.
        const int r = moe_down_rows(a.T, a.H, a.I, FP8);
        if (r == 2) return launch_moe_down<T, FP8, CB, 2, INLINE>(a, 2, s);
        if (r == 4) return launch_moe_down<T, FP8, CB, 4, INLINE>(a, 4, s);
    }
    return launch_moe_down<T, FP8, CB, 1, INLINE>(a, 1, s);
}

constexpr int kMoeMaxKSlices = 8;  // most K slices of the row-shared and panel down projections

// Row groups per wave and K slices of the row-shared down projection for CB token blocks per task.
static int moe_tile_down_rows(int cb, int H) {
    const int r = cb > 4 ? 4 : 2;
    return (H / 16) % (r * kTileWaves) == 0 ? r : 1;
}
static int moe_tile_down_slices(int cb, int H, int I, int max_tasks) {
    const int r = moe_tile_down_rows(cb, H);
    if (r == 1) return 1;
    const int row_tiles = (H / 16) / (r * kTileWaves);
    const int windows = (I / 32) / (cb > 4 ? 2 : 4);
    int skd = 1;
    while (skd < kMoeMaxKSlices && row_tiles * max_tasks * skd < 512 && windows % (skd * 2) == 0) skd *= 2;
    return skd;
}

template <class T, bool FP8, int CB>
static int launch_moe_tile(const MoeArgs &a, int max_tasks, float *obuf, hipStream_t s) {
    // gate/up: two pairs of row groups per wave from five token blocks up (halves the activation re-reads)
    constexpr int P = CB > 4 ? 2 : 1;
    moe_gate_up_tile_kernel<T, FP8, CB, P>
        <<<dim3(a.I / 16 / kTileWaves / P, max_tasks), 256, tile_lds_bytes<CB>(), s>>>(a);
    MLK_LAUNCH_CHECK();
    // down: R row groups per wave; the few output rows (H/16 row groups) are spread over enough
    // workgroups by slicing K, each slice a whole number of windows
    constexpr int R = CB > 4 ? 4 : 2;
    const int groups_h = a.H / 16;
    if (groups_h % (R * kTileWaves) == 0) {
        const int row_tiles = groups_h / (R * kTileWaves);
        const int skd = moe_tile_down_slices(CB, a.H, a.I, max_tasks);
        moe_down_tile_kernel<T, FP8, CB, R><<<dim3(row_tiles, max_tasks, skd), 256, tile_lds_bytes<CB>(), s>>>(a, obuf);
        MLK_LAUNCH_CHECK();
        moe_combine_kernel<T><<<dim3(a.T, (a.H + 1023) / 1024), 256, 0, s>>>(obuf, a.Y, a.topk_ids, a.experts_map, a.K, a.H, a.E, skd);
    } else {
        moe_down_tile_kernel<T, FP8, CB, 1><<<dim3(groups_h / kTileWaves, max_tasks, 1), 256, tile_lds_bytes<CB>(), s>>>(a, obuf);
        MLK_LAUNCH_CHECK();
        moe_combine_kernel<T><<<dim3(a.T, (a.H + 1023) / 1024), 256, 0, s>>>(obuf, a.Y, a.topk_ids, a.experts_map, a.K, a.H, a.E, 1);
    }
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

template <class T, bool FP8>
static int launch_moe_cb(const MoeArgs &a, int cb, int max_tasks, bool inline_align, float *obuf, hipStream_t s) {
    if (inline_align) return launch_moe<T, FP8, 1, true>(a, max_tasks, s);
    const bool tile = moe_tile_path();
    switch (cb) {
        case 1: return launch_moe<T, FP8, 1, false>(a, max_tasks, s);
        case 2: return tile ? launch_moe_tile<T, FP8, 2>(a, max_tasks, obuf, s) : launch_moe<T, FP8, 2, false>(a, max_tasks, s);
        case 3: return tile ? launch_moe_tile<T, FP8, 3>(a, max_tasks, obuf, s) : launch_moe<T, FP8, 3, false>(a, max_tasks, s);
        case 4: return tile ? launch_moe_tile<T, FP8, 4>(a, max_tasks, obuf, s) : launch_moe<T, FP8, 4, false>(a, max_tasks, s);
        case 6: return launch_moe_tile<T, FP8, 6>(a, max_tasks, obuf, s);
        default: return launch_moe_tile<T, FP8, 8>(a, max_tasks, obuf, s);
    }
}

extern template int launch_moe_panel<BF16, true>(const MoeArgs &, int, int, float *, int, bool, hipStream_t);

// Shape of the panel down projection: its grid is (H / 256 row tiles, tasks, K slices), and its kernel comes with a
// short LDS ring (two workgroups per CU, two waves per SIMD) and a long one (one per CU).  Two per CU pay when the
// grid fills them: `pairs` when K slices of at least four 128-wide k windows bring the expected grid (one task per
// active expert; the task list's upper bound counts the tasks a skewed routing adds) to two workgroups per CU
// (Mixtral shape, 256 tokens: 16 x 8 x 4 workgroups, 118 us against 140 us with one per CU and two slices, and 177 us
// with two per CU and two slices, which leaves half the CUs idle).  Otherwise one per CU: slice K while the grid's
// upper bound holds fewer than one and a half workgroups per CU.
// Experiment switch 10: slices + 16 x pairs, in place of this choice.
static void moe_panel_down_shape(int hidden, int inter, int active, int max_tasks, int *slices, bool *pairs) {
    const int row_tiles = hidden / 256, windows = inter / 128, cus = device_cus();
    if (g_tunable[10] > 0) {
        *slices = g_tunable[10] & 15;
        if (*slices < 1) *slices = 1;
        if (*slices > kMoeMaxKSlices) *slices = kMoeMaxKSlices;
        if (*slices > windows) *slices = windows;
        *pairs = (g_tunable[10] >> 4) != 0;
        return;
    }
    int skd = 1;
    while (skd < kMoeMaxKSlices && row_tiles * active * skd < 2 * cus && windows / (skd * 2) >= 4) skd *= 2;
    *pairs = row_tiles * active * skd >= 2 * cus;
    if (*pairs) {
        *slices = skd;
        return;
    }
    skd = 1;
    while (skd < kMoeMaxKSlices && row_tiles * max_tasks * skd * 2 < cus * 3 && windows / (skd * 2) >= 4) skd *= 2;
    *slices = skd;
}
// blocks of 32 tokens in a panel for tasks of up to cb blocks of 16
static int moe_panel_tb32(int cb) { return (cb + 1) / 2 > 4 ? 4 : (cb + 1) / 2; }
// The panel kernels take soft-FP8 weights from five token blocks per task on (more than 64 tokens per pass over an
// expert: the matrix cores, not the weight stream, set the pace there) when the output rows tile in 256.
// Experiment switch 9: 1 keeps the row-shared kernels.
static bool moe_panel_path(int cb, int hidden, bool fp8) { return fp8 && cb >= 5 && hidden % 256 == 0 && g_tunable[9] != 1; }

// How one pass of up to kMoeChunk tokens is run.  The launch code below and mlk_moe_plan() both read it.
enum { kMoePathGemv1 = 0, kMoePathDecodeInline = 1, kMoePathDecode = 2, kMoePathTile = 3, kMoePathPanel = 4 };
struct MoePlan {
    int path;         // kMoePath*
    int cb;           // token blocks per task
    int max_tasks;    // upper bound of the task list (grid dimension)
    int down_r;       // down projection: row groups per wave
    int down_slices;  // down projection: K slices across workgroups
    bool down_pairs;  // panel down projection: two workgroups per CU (shorter LDS ring)
    int down_wk;      // decode down kernel: waves per workgroup; panel down kernel: workgroups per CU
    size_t down_lds;  // decode down kernel: dynamic LDS bytes
};
static MoePlan moe_plan(int tc, int n_experts, int topk, int hidden, int inter, bool fp8) {
    MoePlan pl = {};
    const int n_pairs = tc * topk;
    pl.cb = moe_blocks_per_task(tc, topk, n_experts);
    const int active = n_experts < n_pairs ? n_experts : n_pairs;
    pl.max_tasks = active + n_pairs / (16 * pl.cb);
    pl.down_r = pl.down_slices = 1;
    if (g_moe_gemv1 && tc == 1 && topk <= 16 && (size_t)topk * inter * 2 <= 56 * 1024 &&
        (size_t)hidden * 2 <= 56 * 1024 && (!fp8 || (hidden % 64 == 0 && inter % 64 == 0))) {
        pl.path = kMoePathGemv1;
        return pl;
    }
    const bool inline_align = tc <= 16 && n_pairs <= kDecodePairs;
    if (inline_align) pl.cb = 1;
    if (!inline_align && moe_tile_path() && moe_panel_path(pl.cb, hidden, fp8)) {
        pl.path = kMoePathPanel;
        pl.down_r = 4;
        moe_panel_down_shape(hidden, inter, active, pl.max_tasks, &pl.down_slices, &pl.down_pairs);
        pl.down_wk = pl.down_pairs ? 2 : 1;
        return pl;
    }
    if (!inline_align && pl.cb >= 2 && (moe_tile_path() || pl.cb > 4)) {
        pl.path = kMoePathTile;
        pl.down_r = moe_tile_down_rows(pl.cb, hidden);
        pl.down_slices = moe_tile_down_slices(pl.cb, hidden, inter, pl.max_tasks);
        return pl;
    }
    pl.path = inline_align ? kMoePathDecodeInline : kMoePathDecode;
    if (pl.cb == 1) pl.down_r = pl.down_slices = moe_down_rows(tc, hidden, inter, fp8);
    moe_down_shape(tc, pl.down_r, pl.cb, &pl.down_wk, &pl.down_lds);
    return pl;
}

// Per routed pair and slice for the row-shared and panel kernels, per token and slice for the decode kernels,
// nothing for the single-token kernels; the larger of the two weight kinds, since the workspace query does not
// know which one the call will bring.
static size_t moe_obuf_bytes(int tc, int n_experts, int topk, int hidden, int inter) {
    size_t bytes = 256;
    for (int fp8 = 0; fp8 < 2; ++fp8) {
        const MoePlan pl = moe_plan(tc, n_experts, topk, hidden, inter, fp8 != 0);
        size_t need = 0;
        if (pl.path == kMoePathTile || pl.path == kMoePathPanel)
            need = (size_t)tc * topk * pl.down_slices * hidden * sizeof(float);
        else if (pl.path != kMoePathGemv1)
            need = (size_t)tc * pl.down_slices * hidden * sizeof(float);
        if (need > bytes) bytes = need;
    }
    return bytes;
}

}  // namespace mlk

using namespace mlk;

extern "C" int mlk_moe_plan(int n_tokens, int n_experts, int topk, int hidden, int inter, int w_kind, int32_t *out) {
    MLK_REQUIRE(out != nullptr, "moe plan: null pointer");
    MLK_REQUIRE(n_tokens >= 1 && n_experts >= 1 && n_experts <= kMaxExperts && topk >= 1 && topk <= kMaxTopK,
                "moe plan: sizes out of range");
    MLK_REQUIRE(hidden > 0 && inter > 0 && hidden % 128 == 0 && inter % 128 == 0,
                "moe: hidden and intermediate sizes must be multiples of 128");
    const int tc = n_tokens < kMoeChunk ? n_tokens : kMoeChunk;
    const MoePlan pl = moe_plan(tc, n_experts, topk, hidden, inter, w_kind == MLK_FP8_E4M3);
    out[0] = pl.path;
    out[1] = pl.cb;
    out[2] = pl.max_tasks;
    out[3] = pl.down_r;
    out[4] = pl.down_slices;
    out[5] = pl.down_wk;
    out[6] = (int32_t)pl.down_lds;
    out[7] = (int32_t)sizeof(DecodeTables);
    return MLK_OK;
}

extern "C" void mlk_moe_set_tile_path(int on) {
    g_moe_tile = on & 1;
    g_moe_gemv1 = (on >> 1) & 1 ? 0 : 1;       // bit 1 switches the single-token kernels off
}

extern "C" int mlk_fused_routing_gate(const void *logits, int x_kind, int score_fun, int n_tokens, int n_experts,
                                      int n_groups, int topk_groups, int topk, const void *bias, int renormalize,
                                      int32_t *ids, void *weights, void *stream) {
    MLK_REQUIRE(x_kind == MLK_F16 || x_kind == MLK_BF16, "router: logits must be fp16 or bf16");
    MLK_REQUIRE(score_fun == 0 || score_fun == 1, "router: score function must be 0 (softmax) or 1 (sigmoid)");
    MLK_REQUIRE(n_tokens >= 0, "router: negative token count");
    MLK_REQUIRE(n_experts >= 1 && n_experts <= kMaxExperts, "router: 1..256 experts");
    MLK_REQUIRE(n_groups >= 1 && n_experts % n_groups == 0, "router: n_groups must divide the expert count");
    MLK_REQUIRE(topk_groups >= 1 && topk_groups <= n_groups, "router: topk_groups must be in 1..n_groups");
    MLK_REQUIRE(topk >= 1 && topk <= kMaxTopK && topk <= n_experts, "router: topk must be in 1..min(32, experts)");
    if (n_tokens == 0) return MLK_OK;
    MLK_REQUIRE(logits && ids && weights, "router: null pointer");
    hipStream_t s = (hipStream_t)stream;
    // one, two or four experts per lane: a small expert count does not pay for the register slots of a large one
#define MLK_ROUTER(TT, NE)                                                                                       \
    router_kernel<TT, NE><<<n_tokens, 64, 0, s>>>((const uint16_t *)logits, n_tokens, n_experts, n_groups,       \
                                                  topk_groups, topk, score_fun, (const uint16_t *)bias,          \
                                                  renormalize, ids, (uint16_t *)weights)
    // group counts above 64 also live in the register slots
    const int widest = n_experts > n_groups ? n_experts : n_groups;
    if (x_kind == MLK_F16) {
        if (widest <= 64) MLK_ROUTER(F16, 1);
        else if (widest <= 128) MLK_ROUTER(F16, 2);
        else MLK_ROUTER(F16, 4);
    } else {
        if (widest <= 64) MLK_ROUTER(BF16, 1);
        else if (widest <= 128) MLK_ROUTER(BF16, 2);
        else MLK_ROUTER(BF16, 4);
    }
#undef MLK_ROUTER
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

extern "C" int mlk_moe_align_tokens(const int32_t *topk_ids, int n_pairs, int n_experts, int block,
                                    const int32_t *experts_map, int32_t *sorted_token_ids, int32_t *cumsum_buffer,
                                    int32_t *padded_num_blocks, int32_t *experts_ids, void *stream) {
    MLK_REQUIRE(block == 16, "align: the block size must be 16");
    MLK_REQUIRE(n_experts >= 1 && n_experts <= kMaxExperts, "align: 1..256 experts");
    MLK_REQUIRE(n_pairs >= 0, "align: negative pair count");
    MLK_REQUIRE(sorted_token_ids && cumsum_buffer && padded_num_blocks && experts_ids, "align: null pointer");
    MLK_REQUIRE(n_pairs == 0 || topk_ids, "align: null pointer");
    const int max_blocks = (n_pairs + n_experts * 15 + 15) / 16;
    moe_align_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(topk_ids, n_pairs, n_experts, experts_map, sorted_token_ids,
                                                          cumsum_buffer, padded_num_blocks, experts_ids, max_blocks,
                                                          nullptr, nullptr, 1);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

extern "C" size_t mlk_moe_workspace_bytes(int n_tokens, int n_experts, int topk, int hidden, int inter) {
    // the passes of a call share the workspace: full passes of kMoeChunk tokens and a shorter last one, whose plan
    // (more K slices over fewer pairs) may ask for a different carving
    const int tc = n_tokens < kMoeChunk ? n_tokens : kMoeChunk;
    size_t bytes = carve(nullptr, tc, n_experts, topk, hidden, inter, nullptr);
    const int last = n_tokens > kMoeChunk ? n_tokens % kMoeChunk : 0;
    if (last > 0) {
        const size_t b2 = carve(nullptr, last, n_experts, topk, hidden, inter, nullptr);
        if (b2 > bytes) bytes = b2;
    }
    return bytes;
}

static int experts_compute_impl(const void *w1, const void *w2, const void *x, int n_tokens, int n_experts,
                                int topk, int hidden, int inter, int w_kind, int x_kind,
                                const int32_t *topk_ids, const void *topk_weights,
                                const int32_t *experts_map, const float *w1_scale, const float *w2_scale,
                                void *y, void *workspace, size_t workspace_bytes, void *stream) {
    MLK_REQUIRE(x_kind == MLK_F16 || x_kind == MLK_BF16, "moe: activations must be fp16 or bf16");
    MLK_REQUIRE(n_tokens >= 0, "moe: negative token count");
    MLK_REQUIRE(n_experts >= 1 && n_experts <= kMaxExperts, "moe: 1..256 experts");
    MLK_REQUIRE(topk >= 1 && topk <= kMaxTopK, "moe: topk must be in 1..32");
    MLK_REQUIRE(hidden > 0 && inter > 0 && hidden % 128 == 0 && inter % 128 == 0,
                "moe: hidden and intermediate sizes must be multiples of 128");
    MLK_REQUIRE(hidden <= kMaxScaleK && inter <= kMaxScaleK, "moe: hidden and intermediate sizes up to 32768");
    const bool fp8 = w_kind == MLK_FP8_E4M3;
    if (fp8) MLK_REQUIRE(x_kind == MLK_BF16, "moe: soft-FP8 weights need bf16 activations");
    else MLK_REQUIRE(w_kind == x_kind, "moe: weights and activations must have the same 16-bit type");
    if (n_tokens == 0) return MLK_OK;
    MLK_REQUIRE(w1 && w2 && x && y && topk_ids && topk_weights && workspace, "moe: null pointer");
    MLK_REQUIRE(workspace_bytes >= mlk_moe_workspace_bytes(n_tokens, n_experts, topk, hidden, inter),
                "moe: workspace too small");
    hipStream_t s = (hipStream_t)stream;

    for (int t0 = 0; t0 < n_tokens; t0 += kMoeChunk) {
        const int tc = n_tokens - t0 < kMoeChunk ? n_tokens - t0 : kMoeChunk;
        const int n_pairs = tc * topk;
        const MoePlan pl = moe_plan(tc, n_experts, topk, hidden, inter, fp8);
        const int cb = moe_blocks_per_task(tc, topk, n_experts);
        MoeWorkspace ws;
        carve((uint8_t *)workspace, tc, n_experts, topk, hidden, inter, &ws);
        const int max_padded = n_pairs + n_experts * 15;
        int max_blocks = (max_padded + 15) / 16;
        if (max_blocks < (n_pairs < kDecodePairs ? n_pairs : kDecodePairs)) max_blocks = n_pairs < kDecodePairs ? n_pairs : kDecodePairs;
        const int max_tasks = pl.max_tasks;
        // one token: every routed pair is a GeMV with the activations in LDS
        if (pl.path == kMoePathGemv1) {
            Moe1Args m;
            m.W1 = (const uint8_t *)w1;
            m.W2 = (const uint8_t *)w2;
            m.S1 = w1_scale;
            m.S2 = w2_scale;
            m.X = (const uint16_t *)x + (size_t)t0 * hidden;
            m.Y = (uint16_t *)y + (size_t)t0 * hidden;
            m.Hd = ws.hbuf;
            m.wts = (const uint16_t *)topk_weights + (size_t)t0 * topk;
            m.topk_ids = topk_ids + (size_t)t0 * topk;
            m.experts_map = experts_map;
            m.K = topk;
            m.H = hidden;
            m.I = inter;
            m.E = n_experts;
            // tunables 2..5: G, WK of the gate/up kernel, waves of the down kernel, loads in flight
            int G = g_tunable[2], WK = g_tunable[3], DW = g_tunable[4];
            if (G < 1 || WK < 1 || 2 * G * WK > 16 || (inter / 16) % G) G = 1, WK = 8;
            if (DW < topk || DW > 16) DW = 16;
            DW -= DW % topk;
            m.G = G;
            m.WK = WK;
            m.DW = DW;
            const dim3 g1(inter / (16 * G), topk), g2(hidden / 16);
            const int b1 = 2 * G * WK * 64, b2 = DW * 64;
            const size_t l1 = (size_t)hidden * 2, l2 = (size_t)topk * inter * 2;
#define MLK_MOE1(TT, F8, UU)                                                        \
    do {                                                                            \
        moe_gate_up_gemv1_kernel<TT, F8, UU><<<g1, b1, l1, s>>>(m);                 \
        moe_down_gemv1_kernel<TT, F8, UU><<<g2, b2, l2, s>>>(m);                    \
    } while (0)
#define MLK_MOE1_U(TT, F8)                                                          \
    do {                                                                            \
        const int depth = g_tunable[5] ? g_tunable[5] : (F8 ? 2 : 4);               \
        if (depth == 2) MLK_MOE1(TT, F8, 2);                                        \
        else if (depth == 3) MLK_MOE1(TT, F8, 3);                                   \
        else if (depth == 6) MLK_MOE1(TT, F8, 6);                                   \
        else if (depth == 8) MLK_MOE1(TT, F8, 8);                                   \
        else MLK_MOE1(TT, F8, 4);                                                   \
    } while (0)
            if (fp8) MLK_MOE1_U(BF16, true);
            else if (x_kind == MLK_F16) MLK_MOE1_U(F16, false);
            else MLK_MOE1_U(BF16, false);
#undef MLK_MOE1_U
#undef MLK_MOE1
            MLK_LAUNCH_CHECK();
            continue;
        }
        // decode-sized batches align inside the GeMM kernels; larger ones run the alignment kernel
        const bool inline_align = pl.path == kMoePathDecodeInline;
        if (!inline_align) {
            moe_align_kernel<<<1, 1024, 0, s>>>(topk_ids + (size_t)t0 * topk, n_pairs, n_experts, experts_map,
                                                ws.sorted, ws.cumsum, ws.padded, ws.experts_ids, max_blocks, ws.tasks,
                                                ws.n_tasks, cb);
            MLK_LAUNCH_CHECK();
        }
        MoeArgs a;
        a.W1 = (const uint8_t *)w1;
        a.W2 = (const uint8_t *)w2;
        a.S1 = w1_scale;
        a.S2 = w2_scale;
        a.X = (const uint16_t *)x + (size_t)t0 * hidden;
        a.Y = (uint16_t *)y + (size_t)t0 * hidden;
        a.Hbuf = ws.hbuf;
        a.wts = (const uint16_t *)topk_weights + (size_t)t0 * topk;
        a.sorted = ws.sorted;
        a.tasks = ws.tasks;
        a.n_tasks = ws.n_tasks;
        a.T = tc;
        a.K = topk;
        a.H = hidden;
        a.I = inter;
        a.SB = ws.sb;
        a.n_pairs = n_pairs;
        a.WK = 1;
        a.E = n_experts;
        a.topk_ids = topk_ids + (size_t)t0 * topk;
        a.experts_map = experts_map;
        a.part = ws.obuf;
        a.counters = ws.counters;
        a.n_counters = hidden / 16;
        int rc;
        if (pl.path == kMoePathPanel) {
            const int tb32 = moe_panel_tb32(cb), skd = pl.down_slices;
            const dim3 cgrid(tc, (hidden + 1023) / 1024);
            rc = launch_moe_panel<BF16, true>(a, tb32, max_tasks, ws.obuf, skd, pl.down_pairs, s);
            if (rc != MLK_OK) return rc;
            moe_combine_kernel<BF16><<<cgrid, 256, 0, s>>>(ws.obuf, a.Y, a.topk_ids, a.experts_map, topk, hidden, n_experts, skd);
            MLK_LAUNCH_CHECK();
            continue;
        }
        if (fp8) rc = launch_moe_cb<BF16, true>(a, cb, max_tasks, inline_align, ws.obuf, s);
        else if (x_kind == MLK_F16) rc = launch_moe_cb<F16, false>(a, cb, max_tasks, inline_align, ws.obuf, s);
        else rc = launch_moe_cb<BF16, false>(a, cb, max_tasks, inline_align, ws.obuf, s);
        if (rc != MLK_OK) return rc;
    }
    return MLK_OK;
}

extern "C" int mlk_fused_experts_compute(const void *w1, const void *w2, const void *x, int n_tokens, int n_experts,
                                         int topk, int hidden, int inter, int w_kind, int x_kind,
                                         const int32_t *topk_ids, const void *topk_weights,
                                         const int32_t *experts_map, const float *w1_scale, const float *w2_scale,
                                         void *y, void *workspace, size_t workspace_bytes, void *stream) {
    return experts_compute_impl(w1, w2, x, n_tokens, n_experts, topk, hidden, inter, w_kind, x_kind, topk_ids,
                                topk_weights, experts_map, w1_scale, w2_scale, y, workspace, workspace_bytes, stream);
}

extern "C" int mlk_fused_moe(const void *w1, const void *w2, const void *x, const void *logits, int n_tokens,
                             int n_router_experts, int n_experts, int topk, int hidden, int inter, int w_kind,
                             int x_kind, int score_fun, int n_groups, int topk_groups, const void *bias,
                             int renormalize, const int32_t *experts_map, const float *w1_scale,
                             const float *w2_scale, int32_t *topk_ids, void *topk_weights, void *y, void *workspace,
                             size_t workspace_bytes, void *stream) {
    // the router's own argument checks, whoever routes
    MLK_REQUIRE(x_kind == MLK_F16 || x_kind == MLK_BF16, "router: logits must be fp16 or bf16");
    MLK_REQUIRE(score_fun == 0 || score_fun == 1, "router: score function must be 0 (softmax) or 1 (sigmoid)");
    MLK_REQUIRE(n_tokens >= 0, "router: negative token count");
    MLK_REQUIRE(n_router_experts >= 1 && n_router_experts <= kMaxExperts, "router: 1..256 experts");
    MLK_REQUIRE(n_groups >= 1 && n_router_experts % n_groups == 0, "router: n_groups must divide the expert count");
    MLK_REQUIRE(topk_groups >= 1 && topk_groups <= n_groups, "router: topk_groups must be in 1..n_groups");
    MLK_REQUIRE(topk >= 1 && topk <= kMaxTopK && topk <= n_router_experts, "router: topk must be in 1..min(32, experts)");
    if (n_tokens == 0) return MLK_OK;
    MLK_REQUIRE(logits && topk_ids && topk_weights, "router: null pointer");
    const int rc = mlk_fused_routing_gate(logits, x_kind, score_fun, n_tokens, n_router_experts, n_groups, topk_groups,
                                          topk, bias, renormalize, topk_ids, topk_weights, stream);
    if (rc != MLK_OK) return rc;
    return experts_compute_impl(w1, w2, x, n_tokens, n_experts, topk, hidden, inter, w_kind, x_kind, topk_ids,
                                topk_weights, experts_map, w1_scale, w2_scale, y, workspace, workspace_bytes, stream);
}
