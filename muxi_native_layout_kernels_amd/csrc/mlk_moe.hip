#include "mlk_common.cuh"
using namespace mlk;
extern "C" {
int mlk_fused_routing_gate(const void *, int, int, int, int, int, int, int, const void *, int, int32_t *, void *, void *) { return fail(MLK_ERR_INVALID, "not built yet"); }
int mlk_moe_align_tokens(const int32_t *, int, int, int, const int32_t *, int32_t *, int32_t *, int32_t *, int32_t *, void *) { return fail(MLK_ERR_INVALID, "not built yet"); }
int mlk_fused_experts_compute(const void *, const void *, const void *, int, int, int, int, int, int, int, const void *, const int32_t *, const int32_t *, const int32_t *, const float *, const float *, void *, void *, size_t, void *) { return fail(MLK_ERR_INVALID, "not built yet"); }
size_t mlk_moe_workspace_bytes(int, int, int, int, int) { return 0; }
}
