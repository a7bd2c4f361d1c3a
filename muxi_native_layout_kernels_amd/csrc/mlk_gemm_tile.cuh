// Wave-level building blocks of the narrow GeMM: operand fragments for
// v_mfma_f32_16x16x32_{f16,bf16} straight from the native layouts.
//
// Fragment maps (lane = 16 q + r):
//   weights     lane holds row r, k = 32 t + 8 q .. +7  -> 16 bytes at tile + 16*lane of layout-A
//               (8 bytes at tile + 8*lane for fp8, widened in registers)
//   activations lane holds token r, same k              -> 16 bytes at tile + 16*lane of layout-B,
//               or 16 bytes of row r of a row-major [M, K] matrix
//   accumulator lane holds token r, weight rows 4 q .. 4 q + 3
#pragma once

#include "mlk_common.cuh"

namespace mlk {

// Most threads a workgroup may have for a given number of 16x16 accumulator tiles per wave,
// so that the register file holds the accumulators plus the prefetch ring without spilling.
__host__ __device__ constexpr int max_threads_for_tiles(int ntile) {
    return ntile <= 4 ? 1024 : (ntile <= 8 ? 512 : 256);
}

// One k-tile (32 k) of weights for one row group, as an MFMA operand.
template <bool FP8>
struct WeightFrag {
    u32x4 v;
};
template <>
struct WeightFrag<true> {
    u32x2 v;
};

template <bool FP8>
__device__ __forceinline__ WeightFrag<FP8> load_weight_frag(const uint8_t *rg_base, int kt, int lane) {
    WeightFrag<FP8> f;
    if constexpr (FP8) f.v = ld_stream_u32x2(rg_base + (size_t)kt * 512 + lane * 8);
    else f.v = ld_stream_u32x4(rg_base + (size_t)kt * 1024 + lane * 16);
    return f;
}

// R weight fragments of one k tile -> MFMA operands.  For fp8, `scale[r]` is the (wave-uniform)
// block scale of stream r; one scalar test picks the short power-of-two road for the whole tile.
template <bool FP8, int R>
__device__ __forceinline__ void weight_operands(u32x4 (&a)[R], const WeightFrag<FP8> (&f)[R], const float (&scale)[R]) {
    if constexpr (FP8) {
        bool pow2 = true;
#pragma unroll
        for (int r = 0; r < R; ++r) pow2 = pow2 && scale_is_pow2(scale[r]);
        if (pow2) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t x0, x1, x2, x3;
                fp8x4_to_bf16x4_pow2(f[r].v[0], scale[r], x0, x1);
                fp8x4_to_bf16x4_pow2(f[r].v[1], scale[r], x2, x3);
                a[r] = u32x4{x0, x1, x2, x3};
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t x0, x1, x2, x3;
                fp8x4_to_bf16x4(f[r].v[0], scale[r], x0, x1);
                fp8x4_to_bf16x4(f[r].v[1], scale[r], x2, x3);
                a[r] = u32x4{x0, x1, x2, x3};
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) a[r] = f[r].v;
    }
}

// Store 4 consecutive outputs (weight rows n .. n+3 of one token) as 8 bytes.
template <class T>
__device__ __forceinline__ void store4(uint16_t *p, float a, float b, float c, float d) {
    u32x2 o;
    o[0] = T::from_f32(a) | (T::from_f32(b) << 16);
    o[1] = T::from_f32(c) | (T::from_f32(d) << 16);
    *reinterpret_cast<u32x2 *>(p) = o;
}

}  // namespace mlk
