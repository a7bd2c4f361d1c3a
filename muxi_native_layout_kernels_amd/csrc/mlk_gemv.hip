// Weight-stationary GeMV over layout-A weights: a pure HBM-streaming kernel.
//
// A row group (16 weight rows) is one contiguous run of K*32 bytes (K*16 for
// fp8).  A workgroup owns `G` consecutive row groups; `WK` waves share one row
// group and take its 1 KiB tiles round-robin, so the workgroup always reads a
// contiguous window of G*WK KiB.  Every lane issues 16-byte loads at
// `tile + lane*16` (fully coalesced, non-temporal), keeps `U` of them in flight
// in a register ring, and multiplies by the matching 8 activations read from
// LDS (the activation vector is staged there once per workgroup).  Products
// are accumulated in fp32 with v_dot2; no matrix-core instruction is used.
// Lane partials are folded with cross-lane shuffles, wave partials through
// LDS in a fixed order, so the result is deterministic and needs neither
// atomics nor a zero-filled output.
//
// Algorithmic traffic per call: N*K*sizeof(W) weight bytes (+ 4 bytes per
// 128x128 block of scales) + M*K*2 + M*N*2.
#include "mlk_common.cuh"

namespace mlk {

constexpr int kXsBytes = 48 * 1024;  // LDS window for the staged activations

template <class T, bool FP8, int M, int U>
__global__ void __launch_bounds__(1024)
    gemv_stream_kernel(const uint8_t *__restrict__ A, const uint16_t *__restrict__ X, uint16_t *__restrict__ Y,
                       int n_groups, int K, int KC, float alpha, const uint16_t *__restrict__ bias,
                       const float *__restrict__ scale, int G, int WK) {
    extern __shared__ u32x4 xs[];                 // [M][KC/8] granules of 8 activations
    __shared__ float red[16 * 16 * M];            // [wave][row][m]

    constexpr int TK = FP8 ? 64 : 32;             // k covered by one 1 KiB tile
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, kept scalar
    const int rg_local = wave / WK;
    const int ks = wave - rg_local * WK;
    const int rg = blockIdx.x * G + rg_local;
    const bool active = rg < n_groups;
    const int N = n_groups * 16;
    const int tiles_total = K / TK;
    const int scale_cols = (K + 127) >> 7;

    // lane -> (k octet inside the tile) ; for 16-bit weights the lane holds row lane&15,
    // for fp8 it holds the row pair 2*(lane&7), 2*(lane&7)+1.
    const int oct = FP8 ? (lane >> 3) : (lane >> 4);

    float acc[FP8 ? 2 : 1][M];
#pragma unroll
    for (int a = 0; a < (FP8 ? 2 : 1); ++a)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[a][m] = 0.f;

    ScaleRow srow;
    if (FP8) srow = load_scale_row(scale ? scale + (size_t)((active ? rg : 0) >> 3) * scale_cols : nullptr, scale_cols, lane);

    const u32x4 *arow = reinterpret_cast<const u32x4 *>(A) + (size_t)(active ? rg : 0) * tiles_total * 64 + lane;
    const int stride = WK * 64;                   // u32x4 units between this wave's tiles

    for (int kc0 = 0; kc0 < K; kc0 += KC) {
        const int kc_len = min(KC, K - kc0);
        const int t0 = kc0 / TK;
        const int tiles_here = kc_len / TK;
        const int nt = (active && ks < tiles_here) ? (tiles_here - ks + WK - 1) / WK : 0;
        const u32x4 *ap = arow + (size_t)(t0 + ks) * 64;

        // Register ring of U tiles.  The steady-state loop is branch-free so that the
        // loads stay U deep in flight (the waits become vmcnt(U-1)).
        u32x4 buf[U];
        float sc[U];
        auto issue = [&](int u, int j) {          // j = index among this wave's tiles in the window
            buf[u] = ld_stream_u32x4(ap + (size_t)j * stride);
            if (FP8) sc[u] = scale_at(srow, (t0 + ks + j * WK) >> 1);
        };
        auto consume = [&](int u, int j) {
            u32x4 cur = buf[u];
            const int xg = (ks + j * WK) * (TK / 8) + oct;   // granule of 8 activations
            if (FP8) {
                float s = sc[u];
                uint32_t w0[4], w1[4];
                if (scale_is_pow2(s)) {
                    fp8x4_to_bf16x4_pow2(cur[0], s, w0[0], w0[1]);
                    fp8x4_to_bf16x4_pow2(cur[1], s, w0[2], w0[3]);
                    fp8x4_to_bf16x4_pow2(cur[2], s, w1[0], w1[1]);
                    fp8x4_to_bf16x4_pow2(cur[3], s, w1[2], w1[3]);
                } else {
                    fp8x4_to_bf16x4(cur[0], s, w0[0], w0[1]);
                    fp8x4_to_bf16x4(cur[1], s, w0[2], w0[3]);
                    fp8x4_to_bf16x4(cur[2], s, w1[0], w1[1]);
                    fp8x4_to_bf16x4(cur[3], s, w1[2], w1[3]);
                }
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    u32x4 xv = xs[m * (KC >> 3) + xg];
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        acc[0][m] = T::dot2(w0[d], xv[d], acc[0][m]);
                        acc[FP8 ? 1 : 0][m] = T::dot2(w1[d], xv[d], acc[FP8 ? 1 : 0][m]);
                    }
                }
            } else {
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    u32x4 xv = xs[m * (KC >> 3) + xg];
#pragma unroll
                    for (int d = 0; d < 4; ++d) acc[0][m] = T::dot2(cur[d], xv[d], acc[0][m]);
                }
            }
        };

        // start the weight stream before touching the activations
        const bool full = nt >= U;
        if (full) {
#pragma unroll
            for (int u = 0; u < U; ++u) issue(u, u);
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (u < nt) issue(u, u);
        }

        if (kc0 > 0) __syncthreads();             // everyone is done with the previous window
        const int granules = kc_len >> 3;
        for (int i = threadIdx.x; i < M * granules; i += blockDim.x) {
            int m = i / granules, g = i - m * granules;
            xs[m * (KC >> 3) + g] = *reinterpret_cast<const u32x4 *>(X + (size_t)m * K + kc0 + g * 8);
        }
        __syncthreads();

        if (full) {
            int i = 0;
            for (; i + 2 * U <= nt; i += U) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    consume(u, i + u);
                    issue(u, i + U + u);
                    __builtin_amdgcn_sched_barrier(0);  // keep each refill right behind its consume
                }
            }
            const int rem = nt - i - U;           // 0 .. U-1 tiles still to be fetched
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
    }

    // fold the k octets held by different lanes of the wave
#pragma unroll
    for (int a = 0; a < (FP8 ? 2 : 1); ++a)
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float v = acc[a][m];
            if (FP8) v += lane_xor(v, 8);
            v += lane_xor(v, 16);
            v += lane_xor(v, 32);
            acc[a][m] = v;
        }
    if (FP8) {
        if (lane < 8) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                red[(wave * 16 + 2 * lane) * M + m] = acc[0][m];
                red[(wave * 16 + 2 * lane + 1) * M + m] = acc[FP8 ? 1 : 0][m];
            }
        }
    } else {
        if (lane < 16) {
#pragma unroll
            for (int m = 0; m < M; ++m) red[(wave * 16 + lane) * M + m] = acc[0][m];
        }
    }
    __syncthreads();

    // fold the WK waves of each row group in a fixed order, then the epilogue
    for (int i = threadIdx.x; i < G * 16 * M; i += blockDim.x) {
        int m = i % M;
        int row = (i / M) & 15;
        int gl = i / (16 * M);
        int g = blockIdx.x * G + gl;
        if (g < n_groups) {
            float sum = 0.f;
            for (int w = 0; w < WK; ++w) sum += red[((gl * WK + w) * 16 + row) * M + m];
            int col = g * 16 + row;
            float out = alpha * sum;
            if (bias) out += T::to_f32(bias[col]);
            Y[(size_t)m * N + col] = (uint16_t)T::from_f32(out);
        }
    }
}


// Kernel id 2: the same stream as one uninterrupted run per wave.  The grid is a small multiple of the CU
// count; a workgroup owns a contiguous range of row groups (dealt out evenly) and its W waves take the
// 1 KiB tiles of every row group round-robin, as above.  The register ring of U loads keeps running across
// row-group boundaries, so the only ramp-up and drain of the load pipeline is the one at the start and the
// end of the kernel, and the activation vector is staged in LDS once per workgroup (the whole K, M * K * 2
// bytes).  At a row-group boundary a wave folds its lanes and parks 16 partial sums per token in LDS; the
// waves' partials are added in wave order after the stream has ended.
template <class T, bool FP8, int M, int U, bool MX>
__global__ void __launch_bounds__(1024)
    gemv_persistent_kernel(const uint8_t *__restrict__ A, const uint16_t *__restrict__ X, uint16_t *__restrict__ Y,
                           int n_groups, int K, float alpha, const uint16_t *__restrict__ bias,
                           const float *__restrict__ scale, int nrg_max) {
    extern __shared__ u32x4 xs[];                 // [M][K/8] granules of 8 activations, then red[nrg_max][W][16][M]
    constexpr int TK = FP8 ? 64 : 32;
    constexpr int NA = FP8 ? 2 : 1;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int W = blockDim.x >> 6;
    const int rg0 = (int)((long long)blockIdx.x * n_groups / (int)gridDim.x);
    const int nrg = (int)((long long)(blockIdx.x + 1) * n_groups / (int)gridDim.x) - rg0;
    const int N = n_groups * 16;
    const int tiles = K / TK;
    const int tpw = wave < tiles ? (tiles - wave + W - 1) / W : 0;      // this wave's tiles in every row group
    const int total = nrg * tpw;
    const int scale_cols = (K + 127) >> 7;
    const int oct = FP8 ? (lane >> 3) : (lane >> 4);
    float *red = reinterpret_cast<float *>(xs + (size_t)M * (K >> 3));

    // tile (row group g, index t) sits at A + ((rg0 + g) * tiles + t) * 1 KiB
    const u32x4 *ap = reinterpret_cast<const u32x4 *>(A) + ((size_t)rg0 * tiles + wave) * 64 + lane;
    const long long step = (long long)W * 64;                    // to this wave's next tile
    const long long wrap = ((long long)tiles - (long long)tpw * W) * 64;   // extra step into the next row group
    int i_j = 0;
    u32x4 buf[U];
    auto issue = [&](int u) {
        buf[u] = ld_stream_u32x4(ap);
        ap += step;
        if (++i_j == tpw) {
            i_j = 0;
            ap += wrap;
        }
    };

    ScaleRow srow;
    auto scale_row_of = [&](int g) {
        return load_scale_row(scale ? scale + (size_t)((rg0 + g) >> 3) * scale_cols : nullptr, scale_cols, lane);
    };
    if (FP8) srow = scale_row_of(0);

    float acc[NA][M];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[a][m] = 0.f;
    // MX (soft-FP8 only): the products run on the matrix cores, which leaves the vector ALU to the widening.
    // A 16-byte load gives a lane the k octet o = lane / 8 of the row pair p = lane % 8.  Read as the weight
    // operand of v_mfma_f32_16x16x32_bf16 (lane = 16 q + r holds "row" r, k slot q), the even rows of the
    // pairs form a 16 x 32 operand whose row r is weight row 2 (r % 8) over the octets 2 q + r / 8: rows r and
    // r + 8 are the same weight row on even and odd octets.  The activation operand carries, for token m, the
    // even octets in column 2 m and the odd octets in column 2 m + 1, so D[r][2 m] (r < 8) and D[r][2 m + 1]
    // (r >= 8) are the two halves of one dot product.  A second instruction does the odd rows.  Columns of
    // tokens that do not exist repeat the last token and are never read.
    f32x4 acc_e = {0.f, 0.f, 0.f, 0.f}, acc_o = {0.f, 0.f, 0.f, 0.f};
    const int mx_col = lane & 15, mx_q = lane >> 4;
    const int mx_tok = (mx_col >> 1) < M ? (mx_col >> 1) : M - 1;
    const int mx_x = mx_tok * (K >> 3) + 2 * mx_q + (mx_col & 1);
    int c_j = 0, c_g = 0;
    auto consume = [&](int u) {
        const u32x4 cur = buf[u];
        const int t = wave + c_j * W;                            // tile index inside the row group
        const int xg = t * (TK / 8) + oct;
        if constexpr (MX) {
            const float sc = scale_at(srow, t >> 1);
            uint32_t w0[4], w1[4];
            if (scale_is_pow2(sc)) {
                fp8x4_to_bf16x4_pow2(cur[0], sc, w0[0], w0[1]);
                fp8x4_to_bf16x4_pow2(cur[1], sc, w0[2], w0[3]);
                fp8x4_to_bf16x4_pow2(cur[2], sc, w1[0], w1[1]);
                fp8x4_to_bf16x4_pow2(cur[3], sc, w1[2], w1[3]);
            } else {
                fp8x4_to_bf16x4(cur[0], sc, w0[0], w0[1]);
                fp8x4_to_bf16x4(cur[1], sc, w0[2], w0[3]);
                fp8x4_to_bf16x4(cur[2], sc, w1[0], w1[1]);
                fp8x4_to_bf16x4(cur[3], sc, w1[2], w1[3]);
            }
            const u32x4 xv = xs[mx_x + t * 8];
            acc_e = T::mfma(u32x4{w0[0], w0[1], w0[2], w0[3]}, xv, acc_e);
            acc_o = T::mfma(u32x4{w1[0], w1[1], w1[2], w1[3]}, xv, acc_o);
        } else if (FP8) {
            const float sc = scale_at(srow, t >> 1);
            uint32_t w0[4], w1[4];
            if (scale_is_pow2(sc)) {
                fp8x4_to_bf16x4_pow2(cur[0], sc, w0[0], w0[1]);
                fp8x4_to_bf16x4_pow2(cur[1], sc, w0[2], w0[3]);
                fp8x4_to_bf16x4_pow2(cur[2], sc, w1[0], w1[1]);
                fp8x4_to_bf16x4_pow2(cur[3], sc, w1[2], w1[3]);
            } else {
                fp8x4_to_bf16x4(cur[0], sc, w0[0], w0[1]);
                fp8x4_to_bf16x4(cur[1], sc, w0[2], w0[3]);
                fp8x4_to_bf16x4(cur[2], sc, w1[0], w1[1]);
                fp8x4_to_bf16x4(cur[3], sc, w1[2], w1[3]);
            }
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const u32x4 xv = xs[m * (K >> 3) + xg];
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    acc[0][m] = T::dot2(w0[d], xv[d], acc[0][m]);
                    acc[NA - 1][m] = T::dot2(w1[d], xv[d], acc[NA - 1][m]);
                }
            }
        } else {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const u32x4 xv = xs[m * (K >> 3) + xg];
#pragma unroll
                for (int d = 0; d < 4; ++d) acc[0][m] = T::dot2(cur[d], xv[d], acc[0][m]);
            }
        }
        if (MX && ++c_j == tpw) {
            // the row group is complete for this wave: join the two halves of every dot product, park the sums
            c_j = 0;
            mfma_settle();
            float *dst = red + ((size_t)c_g * W + wave) * 16 * M;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = acc_e[i] + lane_xor(acc_e[i], 0x21);
                const float o = acc_o[i] + lane_xor(acc_o[i], 0x21);
                if ((mx_col & 1) == 0 && (mx_col >> 1) < M && mx_q < 2) {
                    const int pr = 4 * mx_q + i;
                    dst[(2 * pr) * M + (mx_col >> 1)] = e;
                    dst[(2 * pr + 1) * M + (mx_col >> 1)] = o;
                }
            }
            acc_e = f32x4{0.f, 0.f, 0.f, 0.f};
            acc_o = f32x4{0.f, 0.f, 0.f, 0.f};
            ++c_g;
            if (c_g < nrg && ((rg0 + c_g) & 7) == 0) srow = scale_row_of(c_g);
        }
        if (!MX && ++c_j == tpw) {
            // the row group is complete for this wave: fold the k octets held by different lanes, park the sums
            c_j = 0;
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    float v = acc[a][m];
                    if (FP8) v += lane_xor(v, 8);
                    v += lane_xor(v, 16);
                    v += lane_xor(v, 32);
                    acc[a][m] = v;
                }
            float *dst = red + ((size_t)c_g * W + wave) * 16 * M;
            if (FP8) {
                if (lane < 8) {
#pragma unroll
                    for (int m = 0; m < M; ++m) {
                        dst[(2 * lane) * M + m] = acc[0][m];
                        dst[(2 * lane + 1) * M + m] = acc[NA - 1][m];
                    }
                }
            } else if (lane < 16) {
#pragma unroll
                for (int m = 0; m < M; ++m) dst[lane * M + m] = acc[0][m];
            }
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int m = 0; m < M; ++m) acc[a][m] = 0.f;
            ++c_g;
            if (FP8 && c_g < nrg && ((rg0 + c_g) & 7) == 0) srow = scale_row_of(c_g);   // next 128-row block
        }
    };

    // start the weight stream before touching the activations
    const bool full = total >= U;
    if (full) {
#pragma unroll
        for (int u = 0; u < U; ++u) issue(u);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < total) issue(u);
    }
    const int granules = K >> 3;
    for (int i = threadIdx.x; i < M * granules; i += blockDim.x) {
        const int m = i / granules, g = i - m * granules;
        xs[m * granules + g] = *reinterpret_cast<const u32x4 *>(X + (size_t)m * K + g * 8);
    }
    __syncthreads();

    if (full) {
        int i = 0;
        for (; i + 2 * U <= total; i += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                consume(u);
                issue(u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const int rem = total - i - U;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            consume(u);
            if (u < rem) issue(u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < rem) consume(u);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < total) consume(u);
    }
    __syncthreads();

    // add the waves' partials of every row group in wave order, then the epilogue
    const int wsum = W < tiles ? W : tiles;                       // waves that had tiles at all
    for (int i = threadIdx.x; i < nrg * 16 * M; i += blockDim.x) {
        const int m = i % M;
        const int row = (i / M) & 15;
        const int g = i / (16 * M);
        float sum = 0.f;
        for (int w = 0; w < wsum; ++w) sum += red[(((size_t)g * W + w) * 16 + row) * M + m];
        const int col = (rg0 + g) * 16 + row;
        float out = alpha * sum;
        if (bias) out += T::to_f32(bias[col]);
        Y[(size_t)m * N + col] = (uint16_t)T::from_f32(out);
    }
}

template <class T, bool FP8, int M>
static int launch_u(const void *a, const void *x, void *y, int n, int k, float alpha, const void *bias,
                    const float *scale, int block, int G, int U, hipStream_t s) {
    const int W = block / 64;
    const int WK = W / G;
    const int n_groups = n / 16;
    const int grid = (n_groups + G - 1) / G;
    constexpr int TK = FP8 ? 64 : 32;
    int KC = k;
    if ((size_t)M * k * 2 > (size_t)kXsBytes) KC = (kXsBytes / (2 * M)) / TK * TK;
    size_t lds = (size_t)M * KC * 2;
#define MLK_GEMV_LAUNCH(UU)                                                                                   \
    gemv_stream_kernel<T, FP8, M, UU><<<grid, block, lds, s>>>((const uint8_t *)a, (const uint16_t *)x,        \
                                                                  (uint16_t *)y, n_groups, k, KC, alpha,       \
                                                                  (const uint16_t *)bias, scale, G, WK)
    switch (U) {
        case 1: MLK_GEMV_LAUNCH(1); break;
        case 2: MLK_GEMV_LAUNCH(2); break;
        case 4: MLK_GEMV_LAUNCH(4); break;
        case 6: MLK_GEMV_LAUNCH(6); break;
        case 8: MLK_GEMV_LAUNCH(8); break;
        default: return fail(MLK_ERR_INVALID, "gemv: loads in flight (p2) must be 1, 2, 4, 6 or 8");
    }
#undef MLK_GEMV_LAUNCH
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

// LDS of the persistent kernel: the activations of the whole K plus the parked partial sums.
static size_t persistent_lds(int m, int k, int nrg_max, int waves) {
    return (size_t)m * k * 2 + (size_t)nrg_max * waves * 16 * m * sizeof(float);
}

// Grid of kernel id 2 for `per_cu` workgroups per CU, and the largest number of row groups a workgroup gets.
static int persistent_grid(int n_groups, int per_cu, int *nrg_max) {
    long long grid = (long long)device_cus() * per_cu;
    if (grid > n_groups) grid = n_groups;
    if (grid < 1) grid = 1;
    *nrg_max = (int)((n_groups + grid - 1) / grid);
    return (int)grid;
}

template <class T, bool FP8, int M, bool MX = false>
static int launch_persistent(const void *a, const void *x, void *y, int n, int k, float alpha, const void *bias,
                             const float *scale, int block, int per_cu, int U, hipStream_t s) {
    const int n_groups = n / 16;
    int nrg_max = 1;
    const int grid = persistent_grid(n_groups, per_cu, &nrg_max);
    const size_t lds = persistent_lds(M, k, nrg_max, block / 64);
#define MLK_GEMV_P(UU)                                                                                          \
    gemv_persistent_kernel<T, FP8, M, UU, MX><<<grid, block, lds, s>>>((const uint8_t *)a, (const uint16_t *)x,  \
                                                                      (uint16_t *)y, n_groups, k, alpha,         \
                                                                      (const uint16_t *)bias, scale, nrg_max)
    switch (U) {
        case 2: MLK_GEMV_P(2); break;
        case 4: MLK_GEMV_P(4); break;
        case 6: MLK_GEMV_P(6); break;
        case 8: MLK_GEMV_P(8); break;
        default: return fail(MLK_ERR_INVALID, "gemv: loads in flight (p2) must be 2, 4, 6 or 8 for kernel 2");
    }
#undef MLK_GEMV_P
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

template <class T, bool FP8>
static int launch_m(int m, const void *a, const void *x, void *y, int n, int k, float alpha, const void *bias,
                    const float *scale, int block, int G, int U, int kernel_id, hipStream_t s) {
    if (kernel_id == 2 || kernel_id == 3) {
        // the persistent kernel keeps the whole activation vector in LDS; shapes beyond that take kernel 1
        int nrg_max = 1;
        persistent_grid(n / 16, G, &nrg_max);
        if (persistent_lds(m, k, nrg_max, block / 64) <= 64 * 1024 && U >= 2) {
            if constexpr (FP8) {
                if (kernel_id == 3) {
                    switch (m) {
                        case 1: return launch_persistent<T, FP8, 1, true>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                        case 2: return launch_persistent<T, FP8, 2, true>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                        case 3: return launch_persistent<T, FP8, 3, true>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                        case 4: return launch_persistent<T, FP8, 4, true>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                        default: return fail(MLK_ERR_INVALID, "gemv: M must be 1..4");
                    }
                }
            }
            switch (m) {
                case 1: return launch_persistent<T, FP8, 1>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                case 2: return launch_persistent<T, FP8, 2>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                case 3: return launch_persistent<T, FP8, 3>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                case 4: return launch_persistent<T, FP8, 4>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
                default: return fail(MLK_ERR_INVALID, "gemv: M must be 1..4");
            }
        }
        G = 1;
        if (U < 2) U = 2;
    }
    switch (m) {
        case 1: return launch_u<T, FP8, 1>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
        case 2: return launch_u<T, FP8, 2>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
        case 3: return launch_u<T, FP8, 3>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
        case 4: return launch_u<T, FP8, 4>(a, x, y, n, k, alpha, bias, scale, block, G, U, s);
        default: return fail(MLK_ERR_INVALID, "gemv: M must be 1..4");
    }
}

}  // namespace mlk

using namespace mlk;

extern "C" int mlk_gemv_layout_a(const void *a, const void *x, void *y, int m, int n, int k, int a_kind, int x_kind,
                                 float alpha, const void *bias, const float *scale, int block_dim_x, int kernel_id,
                                 int p1, int p2, void *stream) {
    MLK_REQUIRE(m >= 1 && m <= 4, "gemv: M must be 1..4");
    MLK_REQUIRE(n >= 0 && k >= 0, "gemv: negative size");
    MLK_REQUIRE(n % 16 == 0, "GEMV m % 16(at least) must be 0");
    MLK_REQUIRE(k % 32 == 0, "GEMV k % 32(at least) must be 0");
    MLK_REQUIRE(kernel_id == 1 || kernel_id == 2 || kernel_id == 3, "gemv: unknown kernel id");
    MLK_REQUIRE(block_dim_x >= 64 && block_dim_x <= 1024 && block_dim_x % 64 == 0,
                "gemv: BLOCK_DIM_X must be a multiple of 64 in 64..1024");
    if (kernel_id == 1)
        MLK_REQUIRE(p1 >= 1 && (block_dim_x / 64) % p1 == 0, "gemv: row groups per workgroup (p1) must divide the wave count");
    else
        MLK_REQUIRE(p1 >= 1 && p1 <= 16, "gemv: workgroups per CU (p1 of kernel 2) must be 1..16");
    MLK_REQUIRE(x_kind == MLK_F16 || x_kind == MLK_BF16, "gemv: activations must be fp16 or bf16");
    if (n == 0) return MLK_OK;
    MLK_REQUIRE(a && x && y, "gemv: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (a_kind == MLK_FP8_E4M3) {
        MLK_REQUIRE(x_kind == MLK_BF16, "gemv: soft-FP8 weights need bf16 activations");
        MLK_REQUIRE(k % 64 == 0, "gemv: soft-FP8 needs K % 64 == 0");
        MLK_REQUIRE(k <= kMaxScaleK, "gemv: soft-FP8 supports K <= 32768");
        return launch_m<BF16, true>(m, a, x, y, n, k, alpha, bias, scale, block_dim_x, p1, p2, kernel_id, s);
    }
    MLK_REQUIRE(a_kind == x_kind, "gemv: weights and activations must have the same 16-bit type");
    MLK_REQUIRE(scale == nullptr, "gemv: a scale matrix is only meaningful for soft-FP8 weights");
    if (x_kind == MLK_F16) return launch_m<F16, false>(m, a, x, y, n, k, alpha, bias, scale, block_dim_x, p1, p2, kernel_id, s);
    return launch_m<BF16, false>(m, a, x, y, n, k, alpha, bias, scale, block_dim_x, p1, p2, kernel_id, s);
}
