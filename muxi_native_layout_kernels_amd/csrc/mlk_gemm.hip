// Host entry points of the narrow GeMM (the kernels live in mlk_gemm_kernels.cuh and are
// instantiated per operand type in mlk_gemm_f16.hip, mlk_gemm_bf16.hip and mlk_gemm_fp8.hip).
#include <atomic>
#include <mutex>

#include "mlk_gemm_kernels.cuh"

namespace mlk {

constexpr size_t kCounterBytes = 64 * 1024;

// Scratch of mlk_gemm_layout_a_noalloc(): arrival counters and fp32 partials of the cross-workgroup K splits,
// for callers that can neither allocate nor pass a workspace.  One copy per GPU, held until the process ends.
// The array has no initialiser, so it is zero-filled when the code object is loaded onto a device, and the K-split
// kernels leave every counter at zero again when a call ends (the last workgroup to arrive resets its counter):
// nothing has to be cleared at set-up, and the first call may just as well be recorded into a HIP graph that is
// replayed later or thrown away.  The partials need no clearing at all (every slice is written before it is read).
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void *> g_scratch_ptr[64];     // per device: the array's address on that device
static std::mutex g_scratch_mutex;

// Address of `scratch` on the current device, looked up once per device (each GPU holds its own copy of the
// array at its own address).  Host code uses this pointer, never the array's name.
static int static_scratch(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(MLK_ERR_LAUNCH, hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(MLK_ERR_INVALID, "gemm: device index above 63");
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
        if (ptr == nullptr) {
            e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || ptr == nullptr)
                return fail(MLK_ERR_LAUNCH, e != hipSuccess ? hipGetErrorString(e) : "gemm: no address for the static scratch");
            g_scratch_ptr[dev].store(ptr, std::memory_order_release);
        }
    }
    *out = ptr;
    return MLK_OK;
}

// Experiment switches (mlk_set_tunable): [0] rotate the k-tile order per row tile,
// [1] stage row-major activations through LDS, [2]..[5] and [7] shape the fused MoE kernels
// (listed with the declaration of mlk_set_tunable); 0 means automatic for [5], [7] and [8].
int g_tunable[16] = {1, 1, 1, 8, 16, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

extern template int launch_modes<F16, false>(const GemmArgs &, int, int, int, int, int, hipStream_t);
extern template int launch_modes<BF16, false>(const GemmArgs &, int, int, int, int, int, hipStream_t);
extern template int launch_modes<BF16, true>(const GemmArgs &, int, int, int, int, int, hipStream_t);

// kernel id 3 (mlk_panel.hip)
size_t panel_partial_bytes(int m, int n, int sk);
int launch_panel(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, float alpha, const void *bias,
                 const float *scale, int width, int rows, int sk, bool last_round_only, void *counters,
                 size_t counter_bytes, void *partial, size_t partial_bytes, hipStream_t s);

}  // namespace mlk

using namespace mlk;

extern "C" void mlk_set_tunable(int id, int value) {
    if (id >= 0 && id < 16) g_tunable[id] = value;
}

extern "C" size_t mlk_gemm_counter_bytes(void) { return kCounterBytes; }

extern "C" size_t mlk_gemm_workspace_bytes(int m, int n, int p1, int p3) {
    (void)p1;
    int cb = (m + 15) / 16;
    if (cb > 8) cb = 8;                                  // kernel 2 takes up to 128 tokens per weight pass
    if (p3 <= 1) return 0;
    size_t bytes = (size_t)p3 * (size_t)(n / 16) * cb * 1024;
    if (m > 64 && panel_partial_bytes(m, n, p3) > bytes) bytes = panel_partial_bytes(m, n, p3);   // kernel id 3 folds whole panels
    return kCounterBytes + bytes;
}

extern "C" int mlk_gemm_layout_a(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, int x_kind,
                                 int b_mode, int c_mode, float alpha, const void *bias, const float *scale,
                                 int kernel_id, int p1, int p2, int p3, void *workspace, size_t workspace_bytes,
                                 void *stream) {
    MLK_REQUIRE(m >= 0 && n >= 0 && k >= 0, "gemm: negative size");
    MLK_REQUIRE(n % 16 == 0, "gemm: N % 16 must be 0");
    MLK_REQUIRE(k % 32 == 0, "gemm: K % 32 must be 0");
    MLK_REQUIRE(kernel_id == 1 || kernel_id == 2 || kernel_id == 3 || kernel_id == 4 || kernel_id == 5 || kernel_id == 12 || kernel_id == 14 || kernel_id == 16 ||
                    kernel_id == 18,
                "gemm: unknown kernel id");
    MLK_REQUIRE(p1 == 1 || p1 == 2 || p1 == 4 || p1 == 8, "gemm: row groups per wave (p1) must be 1, 2, 4 or 8");
    MLK_REQUIRE(kernel_id == 3 || kernel_id == 5 || (n / 16) % p1 == 0, "gemm: row groups per wave (p1) must divide N/16");
    MLK_REQUIRE(p2 == 1 || p2 == 2 || p2 == 4 || p2 == 8 || p2 == 16, "gemm: waves per workgroup (p2) must be 1, 2, 4, 8 or 16");
    MLK_REQUIRE(p3 >= 1 && p3 <= 64, "gemm: K splits across workgroups (p3) must be 1..64");
    MLK_REQUIRE(x_kind == MLK_F16 || x_kind == MLK_BF16, "gemm: activations must be fp16 or bf16");
    MLK_REQUIRE(b_mode == MLK_B_ROWMAJOR || b_mode == MLK_B_NATIVE, "gemm: bad activation placement");
    MLK_REQUIRE(c_mode == MLK_C_ROWMAJOR || c_mode == MLK_C_NATIVE, "gemm: bad output placement");
    if (b_mode == MLK_B_NATIVE || c_mode == MLK_C_NATIVE) MLK_REQUIRE(m % 16 == 0, "gemm: native B / C need M % 16 == 0");
    if (c_mode == MLK_C_NATIVE) MLK_REQUIRE(n % 32 == 0, "gemm: native C needs N % 32 == 0");
    const bool fp8 = a_kind == MLK_FP8_E4M3;
    if (fp8) {
        MLK_REQUIRE(x_kind == MLK_BF16, "gemm: soft-FP8 weights need bf16 activations");
        MLK_REQUIRE(k <= kMaxScaleK, "gemm: soft-FP8 supports K <= 32768");
    } else {
        MLK_REQUIRE(a_kind == x_kind, "gemm: weights and activations must have the same 16-bit type");
        MLK_REQUIRE(scale == nullptr, "gemm: a scale matrix is only meaningful for soft-FP8 weights");
    }
    if (m == 0 || n == 0) return MLK_OK;
    MLK_REQUIRE(a && b && c, "gemm: null pointer");
    if (kernel_id == 3 || kernel_id == 5) {
        // panel kernel: any number of tokens in one launch; kernel id 5 slices only the panels of the last, partial
        // round of one panel per CU; p1 = row groups per wave (2: 128-row panels, 4: 256-row
        // panels, else chosen from the shape); p2 = tokens per panel (1: 128, 2: 256, else chosen from the shape);
        // p3 = K slices (one slice up to 64 tokens, where the
        // workspace is sized for the narrow kernels)
        MLK_REQUIRE(b_mode == MLK_B_ROWMAJOR && c_mode == MLK_C_ROWMAJOR, "gemm: the panel kernel takes row-major B and C");
        MLK_REQUIRE(k % 128 == 0, "gemm: the panel kernel needs K % 128 == 0");
        uint8_t *ws = (uint8_t *)workspace;
        const size_t part_bytes = workspace_bytes > kCounterBytes ? workspace_bytes - kCounterBytes : 0;
        return launch_panel(a, b, c, m, n, k, fp8 ? MLK_FP8_E4M3 : x_kind, alpha, bias, scale, p2 == 1 ? 128 : (p2 == 2 ? 256 : 0),
                            p1 == 2 ? 128 : (p1 == 4 ? 256 : 0), m > 64 ? p3 : 1, kernel_id == 5, ws, kCounterBytes,
                            ws ? ws + kCounterBytes : nullptr, ws ? part_bytes : 0, (hipStream_t)stream);
    }
    int sk = p3;
    if (sk > k / 32) sk = k / 32 > 0 ? k / 32 : 1;
    const int cb_max = (m + 15) / 16 < 8 ? (m + 15) / 16 : 8;
    if (sk > 1) {
        MLK_REQUIRE(workspace != nullptr, "gemm: a K split across workgroups needs a workspace");
        MLK_REQUIRE((size_t)(n / 16 / p1) * sizeof(int) <= kCounterBytes, "gemm: too many row tiles for the counter region");
        if (kernel_id == 2 && (k / 32) % (sk * kTileKW) != 0) sk = 1;   // kernel 2 splits K in whole windows only
        size_t need = kCounterBytes + (size_t)sk * (size_t)(n / 16) * cb_max * 1024;
        if (workspace_bytes < need) return fail(MLK_ERR_WORKSPACE, "gemm: workspace too small");
    }
    int wk = p2;  // clamped per launch to what registers and LDS allow

    GemmArgs g;
    g.A = (const uint8_t *)a;
    g.B = (const uint16_t *)b;
    g.C = (uint16_t *)c;
    g.bias = (const uint16_t *)bias;
    g.scale = scale;
    g.counters = (int *)workspace;
    g.partial = workspace ? (float *)((uint8_t *)workspace + kCounterBytes) : nullptr;
    g.M_total = m;
    g.N = n;
    g.K = k;
    g.WK = wk;
    g.SK = sk;
    g.alpha = alpha;
    g.rotate = g_tunable[0];
    g.depth = kernel_id >= 12 ? kernel_id - 10 : 0;
    hipStream_t s = (hipStream_t)stream;
    // weight passes of at most 64 tokens; 128 with the row-shared kernel on row-major operands when it tiles
    // the shape with two k tiles per window
    int pass = 64;
    if (kernel_id == 2 && m > 64 && b_mode == MLK_B_ROWMAJOR && c_mode == MLK_C_ROWMAJOR &&
        (n / 16) % (kTileWaves * (p1 >= 2 ? 2 : 1)) == 0 && (k / 32) % (sk * 2) == 0)
        pass = 128;
    for (int c0 = 0; c0 < m; c0 += pass) {
        int mm = m - c0 < pass ? m - c0 : pass;
        g.M = mm;
        g.cb0 = c0 / 16;
        int cb = (mm + 15) / 16;
        // eight row groups per wave exist for one token block, or with row-major B and C
        const int r = (p1 == 8 && cb > 1 && !(b_mode == MLK_B_ROWMAJOR && c_mode == MLK_C_ROWMAJOR)) ? 4 : p1;
        int rc;
        if (fp8) rc = launch_modes<BF16, true>(g, kernel_id, b_mode, c_mode, r, cb, s);
        else if (x_kind == MLK_F16) rc = launch_modes<F16, false>(g, kernel_id, b_mode, c_mode, r, cb, s);
        else rc = launch_modes<BF16, false>(g, kernel_id, b_mode, c_mode, r, cb, s);
        if (rc != MLK_OK) return rc;
    }
    return MLK_OK;
}

extern "C" size_t mlk_gemm_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int mlk_gemm_layout_a_noalloc(const void *a, const void *b, void *c, int m, int n, int k, int a_kind,
                                         int x_kind, int b_mode, int c_mode, float alpha, const void *bias,
                                         const float *scale, int kernel_id, int p1, int p2, int p3, void *stream) {
    void *ws = nullptr;
    if (p3 > 1) {
        MLK_REQUIRE(m >= 0 && n >= 0 && n % 16 == 0, "gemm: N % 16 must be 0");
        if (mlk_gemm_workspace_bytes(m, n, p1, p3) > kStaticScratchBytes)
            return fail(MLK_ERR_WORKSPACE,
                        "gemm: this K split needs more than the 16 MiB of built-in scratch; use fewer splits (p3) "
                        "or mlk_gemm_layout_a with a caller-owned workspace");
        const int rc = static_scratch(&ws);
        if (rc != MLK_OK) return rc;
    }
    return mlk_gemm_layout_a(a, b, c, m, n, k, a_kind, x_kind, b_mode, c_mode, alpha, bias, scale, kernel_id, p1, p2,
                             p3, ws, ws ? kStaticScratchBytes : 0, stream);
}
