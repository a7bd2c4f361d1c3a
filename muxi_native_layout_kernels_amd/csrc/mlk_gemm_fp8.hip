// Narrow GeMM kernels instantiated for soft-FP8 weights with bf16 activations.
#include "mlk_gemm_kernels.cuh"

namespace mlk {
template int launch_modes<BF16, true>(const GemmArgs &, int, int, int, int, int, hipStream_t);
}
