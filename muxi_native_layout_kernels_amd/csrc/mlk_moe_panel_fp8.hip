// Fused-MoE panel kernels instantiated for soft-FP8 weights with bf16 activations.
#include "mlk_moe_panel.cuh"

namespace mlk {
template int launch_moe_panel<BF16, true>(const MoeArgs &, int, int, float *, int, bool, hipStream_t);
}
