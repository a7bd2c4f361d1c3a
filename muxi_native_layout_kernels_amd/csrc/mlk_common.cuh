// Shared device helpers for the gfx950 native-layout kernels.
//
// Everything here is written for CDNA4 only: 64-lane wavefronts, 16-byte
// global loads, v_dot2 / v_mfma 16x16x32 for 16-bit operands and the hardware
// OCP-fp8 converter for the soft-FP8 weights.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mlk.h"

namespace mlk {

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// Experiment switches set through mlk_set_tunable().
extern int g_tunable[16];

// Record an error message for mlk_last_error() and return the code.
int fail(int code, const char *msg);

// Compute units of the current device (cached per device; 256 if the runtime cannot tell).
int device_cus();

#define MLK_REQUIRE(cond, msg)                                                  \
    do {                                                                        \
        if (!(cond)) return ::mlk::fail(MLK_ERR_INVALID, msg);                  \
    } while (0)

#define MLK_LAUNCH_CHECK()                                                      \
    do {                                                                        \
        hipError_t e__ = hipGetLastError();                                     \
        if (e__ != hipSuccess) return ::mlk::fail(MLK_ERR_LAUNCH, hipGetErrorString(e__)); \
    } while (0)

// ---------------------------------------------------------------- conversions
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    _Float16 h = (_Float16)f;
    return (uint32_t)__builtin_bit_cast(unsigned short, h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)b);
}

// Element traits for the two 16-bit activation/output types.
struct F16 {
    static constexpr int kind = MLK_F16;
    __device__ static __forceinline__ float to_f32(uint32_t b) { return f16_bits_to_f32(b); }
    __device__ static __forceinline__ uint32_t from_f32(float f) { return f32_to_f16_bits(f); }
    // acc += a.lo*b.lo + a.hi*b.hi with fp32 accumulation
    __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
    }
    __device__ static __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

struct BF16 {
    static constexpr int kind = MLK_BF16;
    __device__ static __forceinline__ float to_f32(uint32_t b) { return bf16_bits_to_f32(b); }
    __device__ static __forceinline__ uint32_t from_f32(float f) { return f32_to_bf16_bits(f); }
    __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
    }
    __device__ static __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// ------------------------------------------------------------- soft-FP8 widening
// Four e4m3 bytes (one dword, byte 0 = lowest k) -> two dwords of packed bf16
// pairs {k0,k1} and {k2,k3}: W = trunc_bf16(fp32(e4m3) * scale).  The hardware
// converter yields the exact fp32 value of each OCP e4m3 byte; one fp32 multiply
// by the block scale and a byte permute that keeps the upper halves reproduces
// the reference's "widen, multiply by 2^120*scale, drop the low 16 bits"
// (csrc/utils.cuh:80-99) for every non-NaN code and |scale| < 2^8.
__device__ __forceinline__ void fp8x4_to_bf16x4(uint32_t w, float scale, uint32_t &lo, uint32_t &hi) {
    f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    float a0 = a[0] * scale, a1 = a[1] * scale, b0 = b[0] * scale, b1 = b[1] * scale;
    // v_perm_b32 selector: bytes 3,2 of the second source then bytes 3,2 of the first
    lo = __builtin_amdgcn_perm(__float_as_uint(a1), __float_as_uint(a0), 0x07060302u);
    hi = __builtin_amdgcn_perm(__float_as_uint(b1), __float_as_uint(b0), 0x07060302u);
}

// Power-of-two scales (sign 0, mantissa 0, normal exponent) take a shorter road: the scaled
// converter v_cvt_scalef32_pk_bf16_fp8 multiplies by 2^(exponent of the scale) while widening
// two bytes to packed bf16, which is exact - the same bits as the general path - at a fifth of
// the VALU work.  The test is on a wave-uniform value, so the branch is scalar.
__device__ __forceinline__ bool scale_is_pow2(float scale) {
    const uint32_t b = __float_as_uint(scale);
    return (b & 0x807fffffu) == 0u && b != 0u && b != 0x7f800000u;
}
__device__ __forceinline__ void fp8x4_to_bf16x4_pow2(uint32_t w, float scale, uint32_t &lo, uint32_t &hi) {
    lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, scale, false));
    hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, scale, true));
}

// One row of block scales (one fp32 per 128 k) kept in registers: lane l of register i holds
// the scale of k block 64 i + l.  scale_at() fetches a wave-uniform entry with v_readlane, so
// the streaming loops never wait on memory for a scale.  Covers K <= 32768.
constexpr int kMaxScaleK = 32768;
struct ScaleRow {
    float v[4];
};
__device__ __forceinline__ ScaleRow load_scale_row(const float *row, int cols, int lane) {
    ScaleRow s;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int idx = lane + 64 * i;
        s.v[i] = (row != nullptr && idx < cols) ? row[idx] : 1.f;
    }
    return s;
}
__device__ __forceinline__ float scale_at(const ScaleRow &s, int kblock /* wave-uniform */) {
    // four v_readlane and scalar selects: no branch, no vector select
    const int l = kblock & 63, hi = kblock >> 6;
    const int a0 = __builtin_amdgcn_readlane(__float_as_int(s.v[0]), l);
    const int a1 = __builtin_amdgcn_readlane(__float_as_int(s.v[1]), l);
    const int a2 = __builtin_amdgcn_readlane(__float_as_int(s.v[2]), l);
    const int a3 = __builtin_amdgcn_readlane(__float_as_int(s.v[3]), l);
    const int lo = (hi & 1) ? a1 : a0, up = (hi & 1) ? a3 : a2;
    return __int_as_float((hi & 2) ? up : lo);
}

// Wait states between the last MFMA of a block and the first read of its accumulators.  The
// compiler pads this hazard along the fall-through path; when a taken branch follows the MFMA
// block directly, a v_accvgpr_read has been observed to run too early and return the previous
// value of the register (16 wait states cover the 8-pass 16x16x32 instructions).
__device__ __forceinline__ void mfma_settle() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 7\n\ts_nop 7");
    __builtin_amdgcn_sched_barrier(0);
}

// 64-lane xor shuffle of an fp32 through the LDS crossbar (no LDS memory used).
__device__ __forceinline__ float lane_xor(float v, int mask) {
    int lane = __lane_id();
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __float_as_int(v)));
}

// Partial sums exchanged between workgroups of one kernel.  The L2 caches of the eight XCDs are
// not coherent with each other for ordinary accesses; agent-scope atomic accesses are (they are
// issued write-through / always-miss), and unlike an agent-scope fence they do not write back or
// invalidate a whole L2.  64-bit relaxed atomics carry two floats each.  A tile of `cells` quads is
// kept as two planes of 8-byte halves (cell i at [i] and [cells + i]), so that the lanes of one
// access instruction cover whole cache lines; 16 bytes per lane side by side would leave every
// instruction writing half of each line it touches.
__device__ __forceinline__ void st_agent_planar(f32x4 *tile, int cells, int i, f32x4 v) {
    uint64_t *q = reinterpret_cast<uint64_t *>(tile);
    uint64_t lo = (uint64_t)__float_as_uint(v[0]) | ((uint64_t)__float_as_uint(v[1]) << 32);
    uint64_t hi = (uint64_t)__float_as_uint(v[2]) | ((uint64_t)__float_as_uint(v[3]) << 32);
    __hip_atomic_store(q + i, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + cells + i, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 ld_agent_planar(const f32x4 *tile, int cells, int i) {
    const uint64_t *q = reinterpret_cast<const uint64_t *>(tile);
    uint64_t lo = __hip_atomic_load(q + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint64_t hi = __hip_atomic_load(q + cells + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    f32x4 v;
    v[0] = __uint_as_float((uint32_t)lo);
    v[1] = __uint_as_float((uint32_t)(lo >> 32));
    v[2] = __uint_as_float((uint32_t)hi);
    v[3] = __uint_as_float((uint32_t)(hi >> 32));
    return v;
}
// Sum of cell i over `n` slices in slice order; `tile_of(s)` is slice s's tile.  The loads of up to
// eight slices are in flight together (they bypass the caches: a round trip each if issued one by one).
template <class TileOf>
__device__ __forceinline__ f32x4 fold_agent_planar(TileOf tile_of, int n, int cells, int i) {
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < n; s0 += 8) {
        f32x4 t[8];
#pragma unroll
        for (int s = 0; s < 8; ++s)
            if (s0 + s < n) t[s] = ld_agent_planar(tile_of(s0 + s), cells, i);
#pragma unroll
        for (int s = 0; s < 8; ++s)
            if (s0 + s < n) v += t[s];
    }
    return v;
}

__device__ __forceinline__ u32x4 ld_global_u32x4(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ u32x4 ld_stream_u32x4(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ __forceinline__ u32x2 ld_stream_u32x2(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
}

}  // namespace mlk
