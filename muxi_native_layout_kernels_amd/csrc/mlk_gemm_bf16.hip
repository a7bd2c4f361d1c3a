// Narrow GeMM kernels instantiated for bf16 weights and activations.
#include "mlk_gemm_kernels.cuh"

namespace mlk {
template int launch_modes<BF16, false>(const GemmArgs &, int, int, int, int, int, hipStream_t);
}
