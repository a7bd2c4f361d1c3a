/* mlk.h - C ABI of the gfx950 (MI355X) native-layout GeMV / narrow-GeMM / fused-MoE kernels.
 *
 * One shared library, plain pointers and sizes, no torch types.  Every entry
 * point replaces one function that the reference exports to Python through its
 * pybind module (csrc/ffi.cu:32-143); the reference line each one stands in for
 * is cited beside it.  All pointers are DEVICE pointers unless said otherwise,
 * all matrices are dense and contiguous, and every call only enqueues work on
 * `stream` (a hipStream_t passed as void*; NULL = the default stream): nothing
 * is allocated and nothing is synchronised.
 *
 * State the library keeps for the whole process: the last error text (per
 * calling thread); the experiment switches of mlk_set_tunable() and
 * mlk_moe_set_tile_path() (plain ints, not thread-safe: set them before other
 * threads call in, they change what every later call launches); per device,
 * the compute-unit count and which kernels have had their LDS limit raised
 * (both written once, safe to race).
 *
 * Naming follows the reference: weights are "A" [N rows = output features,
 * K reduction], activations are "B" [M tokens, K], outputs are "C" [M, N].
 * (The reference calls these m, k and n.)
 *
 * Return value: 0 on success, a negative MLK_ERR_* otherwise; the text of the
 * last failure is available from mlk_last_error().
 */
#ifndef MLK_H_
#define MLK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLK_OK 0
#define MLK_ERR_INVALID (-1)   /* argument outside what the kernels support  */
#define MLK_ERR_LAUNCH (-2)    /* the HIP runtime refused the launch          */
#define MLK_ERR_WORKSPACE (-3) /* workspace too small                         */

/* element kinds */
#define MLK_F16 0
#define MLK_BF16 1
#define MLK_FP8_E4M3 2 /* soft-FP8 weights: one e4m3 byte per element */

/* output placement of the narrow GeMM */
#define MLK_C_ROWMAJOR 0 /* C[M, N]                               */
#define MLK_C_NATIVE 1   /* layout-C [N/32, ceil(M/16), 4, 16, 8] */

/* activation placement of the narrow GeMM */
#define MLK_B_ROWMAJOR 0 /* B[M, K]                               */
#define MLK_B_NATIVE 1   /* layout-B [K/32, ceil(M/16), 4, 16, 8] */

int mlk_version(void);
const char *mlk_last_error(void);
/* Experiment switches for the tuning scripts (process-wide, not thread-safe):
 *   id 0  rotate the k-tile visiting order of the narrow GeMM per row tile (default 1)
 *   id 1  stage row-major activations of the wave GeMM kernel through LDS when more than
 *         32 tokens share a weight pass (default 1)
 *   id 2, 3  single-token MoE, gate/up kernel: row groups per workgroup and waves splitting K
 *         (defaults 1 and 8; 2 * id2 * id3 <= 16)
 *   id 4  single-token MoE, down kernel: waves per workgroup (default 16)
 *   id 5  single-token MoE: 16-byte loads in flight per wave, 2, 3, 4, 6 or 8 (default 0 = 2 for
 *         soft-FP8 weights, 4 otherwise)
 *   id 7  decode MoE (2..16 tokens), down kernel: row groups per wave = K slices across
 *         workgroups, 1, 2 or 4 (default 0 = 4 for soft-FP8 weights, 1 otherwise)
 *   id 8  fused MoE above 16 tokens: upper limit of the token blocks (of 16) that share one pass over an
 *         expert's weights, 1..8 (default 0 = sized from the expected load of an expert)
 *   id 9  fused MoE, soft-FP8 weights, more than 64 tokens per pass over an expert: 1 keeps the row-shared
 *         kernels instead of the panel kernels (default 0)
 *   10    fused MoE, panel kernels: shape of the down projection, K slices (1..8) + 16 x (two workgroups per
 *         CU on the short LDS ring); 0 (default) = chosen from the sizes and the device's CU count
 * The MoE scan script (kernel_args_scan/moe_scan.py) sweeps ids 2..5, 7, 8 and 10.
 * No counterpart in the reference. */
void mlk_set_tunable(int id, int value);
/* Experiment switches of the fused MoE: bit 0 set (default) = use the row-shared kernels for more
 * than 16 tokens, bit 1 set = do NOT use the single-token GeMV kernels.  Default 1.
 * No counterpart in the reference. */
void mlk_moe_set_tile_path(int on);

/* ------------------------------------------------------------------ relayout
 * Pure permutations of 16-byte (16-bit elements) or 8-byte (fp8) granules;
 * bit-exact, any bit pattern. */

/* [N, K] row-major -> layout-A [N/16, K/8, 16, 8].  elem_size 1 or 2.
 * Stands in for the offline `A.view(m//16,16,k//8,8).permute(0,2,1,3)` of the
 * reference's scripts (benchmark_and_test/gemv_benchmark.py:47-48) and the
 * un-exported device packer csrc/moe_kernels/layout.h:58-99.
 * `batch` independent matrices are processed back to back. */
int mlk_pack_layout_a(const void *src, void *dst, int64_t batch, int n, int k, int elem_size, void *stream);
/* inverse of mlk_pack_layout_a */
int mlk_unpack_layout_a(const void *src, void *dst, int64_t batch, int n, int k, int elem_size, void *stream);

/* B[M, K] row-major (16-bit) -> layout-B [K/32, M/16, 4, 16, 8].
 * Replaces `layoutB`, csrc/layout_b.cu:65-99 (ffi.cu:36).  M % 16 == 0, K % 32 == 0. */
int mlk_layout_b(const void *src, void *dst, int m, int k, void *stream);

/* layout-C [N/32, M/16, 4, 16, 8] (16-bit) -> C[M, N] row-major.
 * Replaces `reLayoutC`, csrc/re_layout_c.cu:63-95 (ffi.cu:37).  Any M % 16 == 0
 * (the reference launches an empty grid when M/16 > 104). */
int mlk_re_layout_c(const void *src, void *dst, int m, int n, void *stream);

/* Swap bytes 1 and 2 of every dword of `nbytes` bytes (nbytes % 4 == 0).
 * Replaces `fp8_weight_repack`, csrc/fp8_weight_repack.cu:44-67 (ffi.cu:92-93);
 * covers the whole tensor (the reference skips partial 256x256 blocks). */
int mlk_fp8_weight_repack(const void *src, void *dst, int64_t nbytes, void *stream);

/* Measurement aid: read `nbytes` (a multiple of 1024) once with the GeMV kernels' access pattern
 * and do nothing else; `workgroups` must divide nbytes/1024, `sink` is a device word that is never
 * written in practice (may be NULL).  Used by bench.py to report the read bandwidth the memory
 * system delivers to a pure streaming kernel next to the 8 TB/s peak.  No counterpart in the reference. */
int mlk_stream_read(const void *src, int64_t nbytes, int block_dim_x, int workgroups, void *sink, void *stream);

/* Measurement aid: `workgroups` workgroups of eight waves; every wave reads four 1 KiB operands from `a` and four from
 * `b` (32 KiB each must be readable: 16-bit values, e.g. the head of a weight and of an activation matrix) and issues
 * iters x 16 v_mfma_f32_32x32x16_bf16 on them, nothing else.  flops = workgroups x 8 x iters x 16 x 32768.  Used by
 * bench.py to report the matrix-core rate the chip sustains on the benchmark's operand values (the power limit lowers
 * the clock under dense random operands) next to the 2.5 PFLOP/s peak.  No counterpart in the reference. */
int mlk_mfma_probe(const void *a, const void *b, int iters, int workgroups, void *sink, void *stream);

/* ---------------------------------------------------------------------- GeMV
 * y[M, N] = T(alpha * x[M, K] . A^T (+ bias[N])), 1 <= M <= 4, fp32 accumulate,
 * A in layout-A.  Replaces `gemv_layoutA` / `gemv_layoutA_wapper`,
 * csrc/gemv_layout_a.cu:17-150 (ffi.cu:65-67, :87-91), which only takes M = 1.
 *
 * a_kind MLK_F16 / MLK_BF16 (x and y have the same kind) or MLK_FP8_E4M3 with
 * x_kind MLK_BF16 and `scale` = fp32 [ceil(N/128), ceil(K/128)] (may be NULL = 1).
 * N % 16 == 0, K % 32 == 0 (K % 64 == 0 for fp8).
 * Launch parameters (what the reference's csv rows select):
 *   block_dim_x  threads per workgroup, 64..1024, multiple of 64
 *   kernel_id    1 = streaming kernel, a workgroup per p1 row groups
 *                2 = the same stream, but the grid is p1 workgroups per CU and each workgroup walks a
 *                    contiguous range of row groups (dealt out evenly) in one uninterrupted stream per wave,
 *                    with the whole activation vector staged in LDS once (falls back to kernel 1 when
 *                    M * K * 2 bytes plus the partial sums exceed 64 KiB of LDS)
 *                3 = kernel 2 with the products on the matrix cores (soft-FP8 weights only; 16-bit weights
 *                    run kernel 2): two v_mfma_f32_16x16x32_bf16 per 1 KiB tile take the even and the odd
 *                    rows, the widening stays on the vector ALU
 *   p1           kernel 1: row groups (of 16 rows) per workgroup: >= 1 and divides both N/16 and
 *                block_dim_x/64; the block_dim_x/64/p1 waves of a row group split K.
 *                kernels 2, 3: workgroups per CU, 1..16
 *   p2           16-byte loads kept in flight per wave: 1, 2, 4, 6 or 8 (kernels 2, 3: not 1)
 */
int mlk_gemv_layout_a(const void *a, const void *x, void *y, int m, int n, int k, int a_kind, int x_kind,
                      float alpha, const void *bias, const float *scale, int block_dim_x, int kernel_id, int p1,
                      int p2, void *stream);

/* --------------------------------------------------------------- narrow GeMM
 * C = T(alpha * B . A^T (+ bias[N])), any M >= 1 (in passes over the weights), A in layout-A, MFMA
 * 16x16x32 (32x32x16 in kernel 3) with fp32 accumulation.
 *
 *   b_mode MLK_B_ROWMAJOR, c_mode MLK_C_ROWMAJOR : `gemm_layoutA` / `_wapper`
 *       csrc/gemm_layout_A.cu:684-787 (ffi.cu:43-45, :74-78) and, with
 *       a_kind MLK_FP8_E4M3 + scale, `gemm_layoutA_soft_fp8` / `_wapper`
 *       csrc/gemm_layout_A_soft_fp8.cu:749-862 (ffi.cu:46-48, :79-83)
 *   b_mode MLK_B_NATIVE,   c_mode MLK_C_ROWMAJOR : `gemm_layoutAB_ContinuousC`
 *       csrc/gemm_layout_ab_continuous_c.cu:1051-1093 (ffi.cu:49-51, :84-86)
 *   b_mode MLK_B_NATIVE,   c_mode MLK_C_NATIVE   : `gemm_layoutABC`
 *       csrc/gemm_layout_abc.cu:754-791 (ffi.cu:38-39, :68-73)
 *
 * With a native B or C, M must be a multiple of 16.  N % 16 == 0, K % 32 == 0
 * (K % 64 == 0 for fp8 weights; N % 32 == 0 for a native C).
 * Launch parameters:
 *   kernel_id 1  wave kernel: every wave owns p1 row groups and gathers its own activations;
 *                p2 = waves per workgroup that split K (1, 2, 4, 8 or 16)
 *   kernel_id 2  row-shared kernel: four waves walk the same k tiles and share the activations
 *                of each k window through LDS (p2 is ignored); falls back to kernel 1 for a
 *                shape it does not tile (N/16 not a multiple of 4 p1, or K/32 not a multiple
 *                of 4 p3).  With row-major B and C it takes more than 64 tokens in passes of up
 *                to 128 (p1 limited to 2) instead of 64
 *   kernel_id 3  panel kernel for prefill-sized token counts (the large-tile `muxi_hgemm_layoutA`
 *                of the reference, csrc/muxi_hgemm_layoutA.cu:10-217, is its counterpart): one launch
 *                for any M; a workgroup computes 256 weight rows x 128 tokens with MFMA 32x32x16,
 *                weights straight from layout-A (two lane swaps per register turn two 16-row tiles
 *                into the 32-row operand), activations shared through LDS.  Row-major B and C,
 *                K % 128 == 0, M * K < 2^31; 16-bit and fp8 weights; p1 = 2: panels of 128 rows (with 128
 *                tokens), 4: of 256 rows; p2 = 1: panels of 128 tokens, 2: 256 rows x 256 tokens; any other
 *                value of p1 or p2: chosen from the shape; p3 = K
 *                slices (useful while 256-row x 128-token panels x p3 stay below the CU count; ignored up to 64 tokens)
 *   kernel_id 4  kernel 1 with one workgroup per CU: the N/16 row groups are dealt out as evenly as
 *                possible, two to four per workgroup (p1 and p3 are ignored).  What one CU can pull
 *                through its memory path bounds these kernels, so for few weight rows an even
 *                deal over all CUs beats a fixed p1.  Up to 64 tokens, N/16 above the CU count and at
 *                most four times it (eight times with soft-FP8 weights, whose activations weigh twice as
 *                much against the weight bytes); 16-bit weights with row-major B and C from one token block on,
 *                soft-FP8 weights or native B / C from 17 tokens on with p2 = 4 or 8 (the activations of
 *                a k window are then shared through LDS by the waves); otherwise the same as kernel 1
 *   kernel_id 5  kernel 3 with the K slices (p3) applied only to the panels that are left over after whole
 *                rounds of one panel per CU: with one workgroup per CU the grid runs in rounds, and a last
 *                round that fills a third of the chip costs as much as a full one; slicing just its panels
 *                p3 ways puts the idle CUs to work without paying the fold on every panel.  The same as
 *                kernel 3 when there is no whole round, and kernel 3 with p3 = 1 when nothing is left over or
 *                when the token tiles of a row tile do not divide an XCD's CUs.  Workspace as for kernel 3
 *   kernel_id 12, 14, 16, 18  kernel 1 with 2, 4, 6 or 8 k tiles in flight per wave instead of the
 *                default depth; honoured for up to 16 tokens with row-major B and C, otherwise
 *                the same as kernel 1
 *   p1 = row groups per wave (1, 2, 4 or 8; 8 means 4 when more than 16 tokens meet a native B or C);
 *   p3 = K splits across workgroups (>= 1; > 1 needs
 *   `workspace`).
 * workspace: device scratch of at least mlk_gemm_workspace_bytes() bytes, only
 * read and written inside the call (contents need not be preserved, but the
 * first `mlk_gemm_counter_bytes()` bytes must be zero before the first call and
 * are left zero by every call).  May be NULL when p3 == 1. */
int mlk_gemm_layout_a(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, int x_kind,
                      int b_mode, int c_mode, float alpha, const void *bias, const float *scale, int kernel_id,
                      int p1, int p2, int p3, void *workspace, size_t workspace_bytes, void *stream);
size_t mlk_gemm_workspace_bytes(int m, int n, int p1, int p3);
size_t mlk_gemm_counter_bytes(void);

/* mlk_gemm_layout_a for callers that can neither allocate device memory nor bring a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments, kernels and results as mlk_gemm_layout_a; the scratch of a K split across
 * workgroups (p3 > 1) lives in a device array built into the library, mlk_gemm_noalloc_scratch_bytes() =
 * 16 MiB per GPU, held until the process ends.  A call whose mlk_gemm_workspace_bytes(m, n, p1, p3) exceeds
 * that returns MLK_ERR_WORKSPACE and launches nothing.  The call allocates and frees nothing.  All calls on
 * one GPU share the array: calls that may overlap (different streams, or graphs replayed side by side) race;
 * order them on one stream.  The first call on a GPU looks up the array's address; nothing is cleared: the
 * array is zero-filled when the library's code is loaded onto the GPU and every call leaves its arrival
 * counters at zero again, so the call may be recorded into a HIP graph from the very first one on. */
int mlk_gemm_layout_a_noalloc(const void *a, const void *b, void *c, int m, int n, int k, int a_kind, int x_kind,
                              int b_mode, int c_mode, float alpha, const void *bias, const float *scale,
                              int kernel_id, int p1, int p2, int p3, void *stream);
size_t mlk_gemm_noalloc_scratch_bytes(void);

/* ----------------------------------------------------------------------- MoE */

/* Router: scores (score_fun 0 = softmax, 1 = sigmoid), optional correction
 * bias for selection, grouped selection, top-K with ties to the lower id.
 * Replaces `fused_routing_gate`, csrc/moe_kernels/fused_gating.cu:5-67 ->
 * fused_topK.h:21-607 (ffi.cu:102-105).  logits [T, E] of kind x_kind,
 * ids int32 [T, K], weights x_kind [T, K] (un-biased scores; renormalised in
 * the weights' own precision when `renormalize` != 0, which the reference
 * leaves to its Python caller, muxi_moe_planC.py:69-70).
 * E <= 256, topk <= 32, n_groups divides E, topk_groups <= n_groups. */
int mlk_fused_routing_gate(const void *logits, int x_kind, int score_fun, int n_tokens, int n_experts,
                           int n_groups, int topk_groups, int topk, const void *bias, int renormalize,
                           int32_t *ids, void *weights, void *stream);

/* Token -> expert-block alignment.  Replaces
 * `batched_routed_activation_indexed_to_expert_block_indexed`,
 * csrc/moe_kernels/fused_experts_compute.cu:6-48 -> moe_align_tokens.h:8-94,
 * moe_align_tokens.cu:5-21 (ffi.cu:106-111).
 *   topk_ids            int32 [n_pairs]           (n_pairs = T * K)
 *   sorted_token_ids    int32 [n_pairs + E*(block-1)]; every slot is written
 *                       (routed pairs ascending inside each expert, sentinel
 *                       n_pairs elsewhere) - no pre-fill needed
 *   cumsum_buffer       int32 [E + 1]; on return cumsum[e] + count[e] for
 *                       e < E and the padded total at [E], as the reference's
 *                       atomic cursors leave it
 *   padded_num_blocks   int32 [1]
 *   experts_ids         int32 [ceil((n_pairs + E*(block-1)) / block)]
 *   experts_map         int32 [E_global] or NULL; -1 drops the pair
 * block must be 16. */
int mlk_moe_align_tokens(const int32_t *topk_ids, int n_pairs, int n_experts, int block,
                         const int32_t *experts_map, int32_t *sorted_token_ids, int32_t *cumsum_buffer,
                         int32_t *padded_num_blocks, int32_t *experts_ids, void *stream);

/* Expert compute from a routing decision: token -> expert-block alignment, grouped
 * gate/up GeMM with SiLU(gate)*up, grouped down GeMM, routing-weighted sum back
 * into token order.  Replaces both overloads of `fused_experts_compute`,
 * csrc/moe_kernels/fused_experts_compute.cu:50-296 (ffi.cu:112-143), which run
 * the alignment themselves (:6-48) before the three compute kernels.
 *   w1 [E, 2I, H] and w2 [E, H, I], each expert slab in layout-A; w_kind
 *   MLK_F16 / MLK_BF16 (= x_kind) or MLK_FP8_E4M3 with x_kind MLK_BF16 and fp32
 *   scales w1_scale [E, 2I/128, H/128], w2_scale [E, H/128, I/128] (NULL = 1)
 *   x [T, H], topk_ids int32 [T*K], topk_weights [T*K] of x_kind,
 *   experts_map int32 [E_global] or NULL (-1 drops the pair),
 *   y [T, H] of x_kind (overwritten; needs no zero fill)
 *   workspace: at least mlk_moe_workspace_bytes() bytes of device scratch
 *   (alignment tables and the SiLU intermediate); contents are not preserved.
 * H % 128 == 0, I % 128 == 0, E <= 256.  Tokens are processed in passes of 256. */
int mlk_fused_experts_compute(const void *w1, const void *w2, const void *x, int n_tokens, int n_experts,
                              int topk, int hidden, int inter, int w_kind, int x_kind, const int32_t *topk_ids,
                              const void *topk_weights, const int32_t *experts_map, const float *w1_scale,
                              const float *w2_scale, void *y, void *workspace, size_t workspace_bytes,
                              void *stream);
size_t mlk_moe_workspace_bytes(int n_tokens, int n_experts, int topk, int hidden, int inter);

/* The whole MoE layer in one call: router, alignment, both grouped GeMMs, weighted sum.  Replaces the call
 * sequence of the reference's Python entry `muxi_moe_planC.fused_moe` (muxi_layout_kernels/muxi_moe_planC.py:44-146:
 * `fused_routing_gate`, the renormalisation in torch, the workspace fills, `fused_experts_compute`).  Arguments
 * as for mlk_fused_routing_gate (logits [T, n_router_experts]; ids / weights are outputs, [T, K]) and
 * mlk_fused_experts_compute (n_experts = expert slabs held locally; differs from n_router_experts only under an
 * experts_map).  Same launches and results as the two calls one after the other; one call instead of two keeps
 * the host's share of a decode step small. */
int mlk_fused_moe(const void *w1, const void *w2, const void *x, const void *logits, int n_tokens,
                  int n_router_experts, int n_experts, int topk, int hidden, int inter, int w_kind, int x_kind,
                  int score_fun, int n_groups, int topk_groups, const void *bias, int renormalize,
                  const int32_t *experts_map, const float *w1_scale, const float *w2_scale, int32_t *topk_ids,
                  void *topk_weights, void *y, void *workspace, size_t workspace_bytes, void *stream);

/* How mlk_fused_experts_compute would run one pass of min(n_tokens, 256) tokens; the launch code reads the same
 * plan.  out[0] = kernel family (0 single-token GeMV kernels, 1 decode kernels that align in-kernel, 2 decode
 * kernels after the alignment kernel, 3 row-shared kernels, 4 panel kernels: soft-FP8 weights with more than 64
 * tokens per pass over an expert), out[1] = token blocks per task, out[2] = upper bound of the task list,
 * out[3] = row groups per wave and out[4] = K slices of the down projection, out[5] = waves and out[6] = dynamic
 * LDS bytes of the decode down kernel (families 1, 2; for family 4 out[5] = workgroups per CU the down kernel is
 * built for, 1 or 2), out[7] = its static LDS bytes.  Everything follows from
 * the sizes alone except out[4] and out[5] of family 4, which also depend on the number of compute units of the current
 * device: for that family the call asks the HIP runtime for it (which initialises the runtime) and assumes 256
 * where there is no GPU, so a plan made on a host without a GPU can name another slice count than a launch on a
 * device with a different CU count uses.  For tests and the tuning scripts; no counterpart in the reference. */
int mlk_moe_plan(int n_tokens, int n_experts, int topk, int hidden, int inter, int w_kind, int32_t *out);

#ifdef __cplusplus
}
#endif
#endif /* MLK_H_ */
