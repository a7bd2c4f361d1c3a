// Relayout kernels: layout-A pack / unpack, layout-B pack, layout-C unpack and
// the fp8 byte repack.  All are pure permutations, one 16-byte (or 8-byte)
// granule per thread, writes coalesced; HBM-bound copies.
#include <atomic>
#include <type_traits>

#include "mlk_common.cuh"

namespace mlk {

// --------------------------------------------------------------- error text
static thread_local char g_err[256] = "";

int fail(int code, const char *msg) {
    int i = 0;
    for (; msg[i] && i < 255; ++i) g_err[i] = msg[i];
    g_err[i] = 0;
    return code;
}

int device_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev >= 0 && dev < 64) {
        const int hit = cached[dev].load(std::memory_order_relaxed);
        if (hit > 0) return hit;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

// One granule of 8 elements: G = uint4 for 16-bit elements, uint2 for bytes.
//
// layout-A: dst granule ((g * K/8 + o) * 16 + r)  <-  src granule (16 g + r) * K/8 + o
template <typename G, bool PACK>
__global__ void __launch_bounds__(256) layout_a_kernel(const G *__restrict__ src, G *__restrict__ dst, int64_t total,
                                                       int n, int octets) {
    int64_t per_mat = (int64_t)n * octets;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        int64_t mat = i / per_mat;
        int64_t j = i - mat * per_mat;          // index in native order
        int r = (int)(j & 15);
        int64_t go = j >> 4;
        int o = (int)(go % octets);
        int64_t g = go / octets;
        int64_t rm = (g * 16 + r) * octets + o;  // index in row-major order
        if (PACK) dst[i] = src[mat * per_mat + rm];
        else dst[mat * per_mat + rm] = src[i];
    }
}

// The same permutation in whole cache lines, for K % 64 == 0: a wave moves 8 rows x 8 octets, so that on the
// row-major side every row contributes 8 consecutive granules (a 128-byte line of 16-bit elements) and on the
// native side every octet contributes rows 8 h .. 8 h + 7 (again a full line); the index arithmetic is done
// once per wave and per KiB instead of per granule.  task = ((row group) * 2 + h) * K/64 + octet block, the
// row groups of a batch of matrices counted through.
template <typename G, bool PACK>
__global__ void __launch_bounds__(256) layout_a_lines_kernel(const G *__restrict__ src, G *__restrict__ dst, uint32_t tasks,
                                                             int octets) {
    const int lane = threadIdx.x & 63;
    const int oo = lane & 7, rr = lane >> 3;
    const uint32_t blocks = (uint32_t)octets >> 3;
    const uint32_t wave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (uint32_t t = wave; t < tasks; t += gridDim.x * 4) {
        const uint32_t ob = t % blocks, x = t / blocks;
        const uint32_t h = x & 1;
        const int64_t rg = x >> 1;
        const int64_t rm = (rg * 16 + 8 * h + rr) * octets + ob * 8 + oo;
        const int64_t nat = (rg * octets + ob * 8 + oo) * 16 + 8 * h + rr;
        // every granule is read once and written once: non-temporal both ways
        using V = typename std::conditional<sizeof(G) == 16, u32x4, u32x2>::type;
        const V *s = reinterpret_cast<const V *>(src);
        V *d = reinterpret_cast<V *>(dst);
        if (PACK) __builtin_nontemporal_store(__builtin_nontemporal_load(s + rm), d + nat);
        else __builtin_nontemporal_store(__builtin_nontemporal_load(s + nat), d + rm);
    }
}

// layout-B / layout-C: native granule ((c * M/16 + g) * 64 + 16 q + r) <-> row-major
// granule (16 g + r) * K/8 + 4 c + q.  PACK: row-major -> native (layoutB);
// !PACK: native -> row-major (reLayoutC).  The thread index always runs over
// the destination so stores are coalesced.
template <bool PACK>
__global__ void __launch_bounds__(256) layout_b_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                       int64_t total, int mgroups, int octets) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        if (PACK) {
            int r = (int)(i & 15);
            int q = (int)((i >> 4) & 3);
            int64_t cg = i >> 6;
            int g = (int)(cg % mgroups);
            int64_t c = cg / mgroups;
            dst[i] = src[((int64_t)g * 16 + r) * octets + c * 4 + q];
        } else {
            int64_t row = i / octets;
            int oct = (int)(i - row * octets);
            int g = (int)(row >> 4), r = (int)(row & 15);
            int c = oct >> 2, q = oct & 3;
            dst[i] = src[(((int64_t)c * mgroups + g) << 6) + q * 16 + r];
        }
    }
}

__global__ void __launch_bounds__(256) fp8_repack_kernel(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                         int64_t ndwords) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ndwords;
         i += (int64_t)gridDim.x * blockDim.x) {
        uint32_t w = src[i];
        // bytes [b0, b1, b2, b3] -> [b0, b2, b1, b3]
        dst[i] = __builtin_amdgcn_perm(w, w, 0x03010200u);
    }
}

// The same permutation on 16 bytes per thread (both pointers 16-byte aligned): four dwords per load and per
// store instruction, non-temporal both ways since nothing is read twice.
__global__ void __launch_bounds__(256) fp8_repack16_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                           int64_t nquads) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nquads;
         i += (int64_t)gridDim.x * blockDim.x) {
        u32x4 w = __builtin_nontemporal_load(src + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = __builtin_amdgcn_perm(w[j], w[j], 0x03010200u);
        __builtin_nontemporal_store(w, dst + i);
    }
}

// Matrix-core yardstick: every wave takes four 32-row operands from `a` and four from `b` (16 bytes per lane each, read
// once) and issues iters x 16 v_mfma_f32_32x32x16_bf16 on them, eight waves per workgroup, nothing else in the loop and
// nothing stored.  What it measures is the rate the chip sustains on those operand VALUES: with zeros the clock stays at
// its maximum, with the dense random values of a real product the power limit pulls it down by a third.
__global__ void __launch_bounds__(512) mfma_probe_kernel(const u32x4 *__restrict__ a, const u32x4 *__restrict__ b, int iters,
                                                         uint32_t *__restrict__ sink) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    u32x4 x[4], y[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[i] = a[(wave * 4 + i) * 64 + lane];
        y[i] = b[(wave * 4 + i) * 64 + lane];
    }
    f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = BF16::mfma32(x[2 * r + i], y[j], acc[i][j]);
    }
    mfma_settle();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) s += acc[i][j][0];
    if (sink != nullptr && __float_as_uint(s) == 0x7fc12345u) *sink = 1;      // a NaN payload the products never make
}

// Pure streaming read with the access pattern of the GeMV kernels (1 KiB tiles, 16 bytes per
// lane, non-temporal, U loads in flight per wave): measures what the memory system delivers to
// a kernel that does nothing else.  The xor of everything read is compared with a value the
// data never produces, so the loads cannot be optimised away and nothing is written.
template <int U>
__global__ void __launch_bounds__(1024) stream_read_kernel(const u32x4 *__restrict__ src, int64_t tiles_per_wg,
                                                           uint32_t *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const u32x4 *base = src + (size_t)blockIdx.x * tiles_per_wg * 64 + lane;
    const int nt = wave < tiles_per_wg ? (int)((tiles_per_wg - wave + waves - 1) / waves) : 0;
    u32x4 acc = {0u, 0u, 0u, 0u};
    u32x4 buf[U];
    auto ld = [&](int j) { return ld_stream_u32x4(base + (size_t)(wave + (int64_t)j * waves) * 64); };
    if (nt >= U) {
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = ld(u);
        int i = 0;
        for (; i + 2 * U <= nt; i += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                acc ^= buf[u];
                buf[u] = ld(i + U + u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const int rem = nt - i - U;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc ^= buf[u];
            if (u < rem) buf[u] = ld(i + U + u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < rem) acc ^= buf[u];
    } else {
        for (int j = 0; j < nt; ++j) acc ^= ld(j);
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) sink[threadIdx.x & 63] = acc[0];
}

static inline int grid_for(int64_t total) {
    int64_t blocks = (total + 255) / 256;
    const int64_t cap = 256 * 32;  // 32 workgroups per CU is plenty for a copy
    return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace mlk

using namespace mlk;

extern "C" {

int mlk_version(void) { return 1; }
const char *mlk_last_error(void) { return g_err; }

static int layout_a_common(const void *src, void *dst, int64_t batch, int n, int k, int elem_size, void *stream,
                           bool pack) {
    MLK_REQUIRE(batch >= 0 && n >= 0 && k >= 0, "layout-A: negative size");
    MLK_REQUIRE(n % 16 == 0 && k % 8 == 0, "layout-A: N % 16 and K % 8 must be 0");
    MLK_REQUIRE(elem_size == 1 || elem_size == 2, "layout-A: element size must be 1 or 2");
    int64_t total = batch * (int64_t)n * (k / 8);
    if (total == 0) return MLK_OK;
    MLK_REQUIRE(src && dst, "layout-A: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const int64_t tasks = total / 64;
    if ((k / 8) % 8 == 0 && tasks < (int64_t)1 << 31) {
        int grid = grid_for(tasks * 64);
        if (elem_size == 2) {
            if (pack) layout_a_lines_kernel<uint4, true><<<grid, 256, 0, s>>>((const uint4 *)src, (uint4 *)dst, (uint32_t)tasks, k / 8);
            else layout_a_lines_kernel<uint4, false><<<grid, 256, 0, s>>>((const uint4 *)src, (uint4 *)dst, (uint32_t)tasks, k / 8);
        } else {
            if (pack) layout_a_lines_kernel<uint2, true><<<grid, 256, 0, s>>>((const uint2 *)src, (uint2 *)dst, (uint32_t)tasks, k / 8);
            else layout_a_lines_kernel<uint2, false><<<grid, 256, 0, s>>>((const uint2 *)src, (uint2 *)dst, (uint32_t)tasks, k / 8);
        }
        MLK_LAUNCH_CHECK();
        return MLK_OK;
    }
    int grid = grid_for(total);
    if (elem_size == 2) {
        if (pack) layout_a_kernel<uint4, true><<<grid, 256, 0, s>>>((const uint4 *)src, (uint4 *)dst, total, n, k / 8);
        else layout_a_kernel<uint4, false><<<grid, 256, 0, s>>>((const uint4 *)src, (uint4 *)dst, total, n, k / 8);
    } else {
        if (pack) layout_a_kernel<uint2, true><<<grid, 256, 0, s>>>((const uint2 *)src, (uint2 *)dst, total, n, k / 8);
        else layout_a_kernel<uint2, false><<<grid, 256, 0, s>>>((const uint2 *)src, (uint2 *)dst, total, n, k / 8);
    }
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

int mlk_pack_layout_a(const void *src, void *dst, int64_t batch, int n, int k, int elem_size, void *stream) {
    return layout_a_common(src, dst, batch, n, k, elem_size, stream, true);
}

int mlk_unpack_layout_a(const void *src, void *dst, int64_t batch, int n, int k, int elem_size, void *stream) {
    return layout_a_common(src, dst, batch, n, k, elem_size, stream, false);
}

int mlk_layout_b(const void *src, void *dst, int m, int k, void *stream) {
    MLK_REQUIRE(m >= 0 && k >= 0, "layoutB: negative size");
    MLK_REQUIRE(m % 16 == 0, "n must be a multiple of 16");
    MLK_REQUIRE(k % 32 == 0, "k must be a multiple of 32");
    int64_t total = (int64_t)m * (k / 8);
    if (total == 0) return MLK_OK;
    MLK_REQUIRE(src && dst, "layoutB: null pointer");
    layout_b_kernel<true><<<grid_for(total), 256, 0, (hipStream_t)stream>>>((const uint4 *)src, (uint4 *)dst, total,
                                                                           m / 16, k / 8);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

int mlk_re_layout_c(const void *src, void *dst, int m, int n, void *stream) {
    MLK_REQUIRE(m >= 0 && n >= 0, "reLayoutC: negative size");
    MLK_REQUIRE(m % 16 == 0, "n must be a multiple of 16");
    MLK_REQUIRE(n % 32 == 0, "m must be a multiple of 32");
    int64_t total = (int64_t)m * (n / 8);
    if (total == 0) return MLK_OK;
    MLK_REQUIRE(src && dst, "reLayoutC: null pointer");
    layout_b_kernel<false><<<grid_for(total), 256, 0, (hipStream_t)stream>>>((const uint4 *)src, (uint4 *)dst, total,
                                                                            m / 16, n / 8);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

int mlk_stream_read(const void *src, int64_t nbytes, int block_dim_x, int workgroups, void *sink, void *stream) {
    MLK_REQUIRE(nbytes >= 0 && nbytes % 1024 == 0, "stream_read: byte count must be a multiple of 1024");
    MLK_REQUIRE(block_dim_x >= 64 && block_dim_x <= 1024 && block_dim_x % 64 == 0,
                "stream_read: threads per workgroup must be a multiple of 64 in 64..1024");
    MLK_REQUIRE(workgroups >= 1, "stream_read: at least one workgroup");
    if (nbytes == 0) return MLK_OK;
    MLK_REQUIRE(src, "stream_read: null pointer");
    int64_t tiles = nbytes / 1024;
    MLK_REQUIRE(tiles % workgroups == 0, "stream_read: the workgroup count must divide the number of 1 KiB tiles");
    stream_read_kernel<4><<<workgroups, block_dim_x, 0, (hipStream_t)stream>>>((const u32x4 *)src, tiles / workgroups,
                                                                              (uint32_t *)sink);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

int mlk_mfma_probe(const void *a, const void *b, int iters, int workgroups, void *sink, void *stream) {
    MLK_REQUIRE(a && b, "mfma_probe: null pointer");
    MLK_REQUIRE(iters >= 0 && workgroups >= 1, "mfma_probe: iterations >= 0, at least one workgroup");
    mfma_probe_kernel<<<workgroups, 512, 0, (hipStream_t)stream>>>((const u32x4 *)a, (const u32x4 *)b, iters, (uint32_t *)sink);
    MLK_LAUNCH_CHECK();
    return MLK_OK;
}

int mlk_fp8_weight_repack(const void *src, void *dst, int64_t nbytes, void *stream) {
    MLK_REQUIRE(nbytes >= 0 && nbytes % 4 == 0, "fp8_weight_repack: byte count must be a multiple of 4");
    if (nbytes == 0) return MLK_OK;
    MLK_REQUIRE(src && dst, "fp8_weight_repack: null pointer");
    int64_t nd = nbytes / 4;
    const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
    const int64_t nq = aligned ? nd / 4 : 0;
    if (nq > 0) {
        fp8_repack16_kernel<<<grid_for(nq), 256, 0, (hipStream_t)stream>>>((const u32x4 *)src, (u32x4 *)dst, nq);
        MLK_LAUNCH_CHECK();
    }
    if (nd > nq * 4) {      // the last one to three dwords, or everything when a pointer is not 16-byte aligned
        fp8_repack_kernel<<<grid_for(nd - nq * 4), 256, 0, (hipStream_t)stream>>>((const uint32_t *)src + nq * 4,
                                                                                  (uint32_t *)dst + nq * 4, nd - nq * 4);
        MLK_LAUNCH_CHECK();
    }
    return MLK_OK;
}

}  // extern "C"
