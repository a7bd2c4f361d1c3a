// Panel main loop with LDS as the only prefetch buffer: a workgroup of four waves multiplies 256 weight rows (each
// wave 64: two pairs of row groups) with TB blocks of 32 token rows over a run of k32 slabs, v_mfma_f32_32x32x16.
//
// Why a second loop beside mlk_panel_loop.cuh: that one keeps weights two k windows ahead in registers and takes a
// whole SIMD's register file, so a SIMD runs one wave, and everything that wave issues besides its MFMAs - loads, LDS
// reads and, with soft-FP8 weights, two VALU instructions per weight to widen them - is time the matrix core
// stands still.  Here nothing waits in registers: a k32 slab of the panel is copied into LDS by buffer loads with the
// LDS bit (no register, no ds_write), four slabs deep, and a workgroup fits in 256 registers and 64 KiB (soft-FP8;
// 16-bit weights: 96 KiB), so that two workgroups share a CU and the widening, the LDS reads and the waits of one
// wave go on under the products of the other wave on its SIMD.
//
// Slab layout (16-byte granules): weight tile 4 w + r (wave w, its row group r) at TG (4 w + r), TG = 32 (fp8: 16 rows
// x 32 k x 1 byte as it lies in layout A) or 64; then token chunk c (16 tokens x 32 k) at 16 TG + 64 c, token t's octet o
// at granule 4 t + (o ^ (t / 4 % 4)): four lanes of a load cover 64 consecutive bytes of a token row, and the 16 lanes
// that read one octet of 16 tokens for an operand hit 16 different bank groups.
// Loads per wave and slab: its own weight tiles (fp8: two loads, each the tiles of a pair of row groups, 32 lanes per tile;
// 16-bit: four, addressed by the thread id alone) and two token chunks (chunk w and w + 4; with three blocks of tokens the
// waves 2 and 3 fetch their first chunk twice, which keeps the count of loads in flight equal in all waves).
// Operands: lane 32 g + i reads row i % 16 of tile i / 16 of the pair, k octet 2 h + g of half step h (8 bytes of fp8,
// widened in registers, or 16 bytes), and token i of a block likewise from its two chunks.
//
// While slab s is multiplied, slab s + 1 is complete and published, slab s + 2 is landing, and the loads of slab s + 3
// go out into the buffer slab s - 1 has left; one wait (this wave's loads of slab s + 2) and one bare s_barrier per slab
// (the fence of __syncthreads() would wait for every load in flight).  The operands of the first half step of slab
// s + 1 are read before that barrier.
#pragma once

#include <type_traits>

#include "mlk_tile.cuh"

namespace mlk {

template <int N>
__device__ __forceinline__ void wait_vmcnt_le() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x70 | 0xF00);
}
__device__ __forceinline__ void bare_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <bool FP8, int TB, int RING_ = 4>
struct PanelLdsShape {
    static constexpr int TG = FP8 ? 32 : 64;                 // granules of a weight tile
    static constexpr int NCH = 2 * TB;                       // token chunks of 16
    static constexpr int BOFF = 16 * TG;                     // first token chunk
    static constexpr int SLAB = BOFF + NCH * 64;
    static constexpr int RING = RING_;
    static constexpr size_t lds_bytes = (size_t)RING * SLAB * 16;
    static constexpr int NA = FP8 ? 2 : 4;                   // weight loads per wave and slab
    static constexpr int NLOAD = NA + 2;                     // waves whose second chunk does not exist: one less
};

// acc[pr][tb] += rows of pair pr x the tokens of block tb over the slabs slab0 .. slab0 + nslab - 1.
//   abase[r]     wave-uniform start of row group r of this wave (r = 2 pr, 2 pr + 1 form pair pr; fp8: both inside 4 GiB
//                of abase[2 pr])
//   srow[pr]     soft-FP8 block scales of the 128-row block that holds pair pr
//   row_off(j)   element offset in B of the row that token slot j of the panel reads (any valid row for slots that hold
//                no token)
template <class T, bool FP8, int TB, int RING = 4>
struct PanelLoopLds {
    using S = PanelLdsShape<FP8, TB, RING>;

    // The loads of one wave for slab `slab` (k = 32 slab .. + 31) into ring buffer `buf`.
    //   abase[r]   wave-uniform start of row group r of this wave in layout A
    //   a_voff     fp8: per-lane byte offset of lane's 16 bytes from abase[2 p] for the load of pair p (the two tiles of a pair
    //              travel in one instruction, 32 lanes each)
    //   b_voff[i]  per-lane byte offset from B of this lane's 16 bytes of chunk load i at k = 0
    __device__ static __forceinline__ void issue(const uint8_t *const *abase, const uint32_t *a_voff, const uint16_t *B,
                                                    const uint32_t *b_voff, int wave, int slab, int buf) {
        extern __shared__ u32x4 win[];
        const int dst = buf * S::SLAB;
        if constexpr (FP8) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)abase[2 * p], 0, 0xffffffffu, 0x00020000);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, win + dst + (4 * wave + 2 * p) * S::TG, 16, a_voff[p], slab * 512, 0, 0);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)abase[r], 16, 0xffffffffu, 1 << 23);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, win + dst + (4 * wave + r) * S::TG, 16, 0, slab * 1024, 0, 0);
            }
        }
        __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, 0xffffffffu, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, win + dst + S::BOFF + wave * 64, 16, b_voff[0], slab * 64, 0, 0);
        if (wave + 4 < S::NCH)                                   // wave-uniform
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, win + dst + S::BOFF + (wave + 4) * 64, 16, b_voff[1], slab * 64, 0, 0);
    }


    template <class RowOff>
    __device__ static __forceinline__ void run(f32x16 (&acc)[2][TB], const uint8_t *const (&abase)[4], const ScaleRow (&srow)[2],
                                               const uint16_t *__restrict__ B, RowOff row_off, int slab0, int nslab, u32x4 *win) {
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        uint32_t a_voff[2] = {0, 0}, b_voff[2];
        if constexpr (FP8) {
#pragma unroll
            for (int p = 0; p < 2; ++p)
                a_voff[p] = (lane >> 5 ? (uint32_t)(abase[2 * p + 1] - abase[2 * p]) : 0u) + (lane & 31) * 16;
        }
        {
            const int t = lane >> 2, oct = (lane & 3) ^ ((t >> 2) & 3);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int chunk = (wave + 4 * i < S::NCH) ? wave + 4 * i : wave;      // the second one may not exist
                b_voff[i] = row_off(chunk * 16 + t) * 2u + oct * 16;
            }
        }
        // operand reads, first half step (second: weights + 32 granules of 16 bytes / + 32 * 8 bytes, tokens ^ 2)
        const int g = lane >> 5, i32 = lane & 31, t16 = i32 & 15, hi = i32 >> 4;
        const int a_idx = FP8 ? ((4 * wave + hi) * 64 + g * 16 + t16)        // in 8-byte units; + 128 pr, + 32 h
                              : ((4 * wave + hi) * 64 + g * 16 + t16);       // in granules;     + 128 pr, + 32 h
        const int b_idx = S::BOFF + hi * 64 + 4 * t16 + (g ^ ((t16 >> 2) & 3));                  // + 128 tb, ^ 2 h

        typedef typename std::conditional<FP8, u32x2, u32x4>::type AFrag;
        AFrag a0[2], a1[2];
        u32x4 b0[TB], b1[TB];
        auto rd = [&](AFrag (&a)[2], u32x4 (&b)[TB], int buf, int hs) {
            const u32x4 *src = win + buf * S::SLAB;
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
                if constexpr (FP8) a[pr] = reinterpret_cast<const u32x2 *>(src)[a_idx + 128 * pr + 32 * hs];
                else a[pr] = src[a_idx + 128 * pr + 32 * hs];
            }
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) b[tb] = src[(b_idx ^ (hs * 2)) + 128 * tb];
        };
        // Soft-FP8: the operands of a half step are widened while the products of the half step before it run (the
        // scheduling pattern below puts five or six conversion instructions between two MFMAs), so that a wave is a
        // uniform mix of both and the two waves of a SIMD - from two workgroups, in no fixed phase to each other - fill
        // the matrix core and the vector ALU at the same time.  With the conversions of a half step in one block in
        // front of its products, two waves that happen to run in step convert at the same time and multiply at the
        // same time, and the layer takes the sum of both (measured: 1,870 cycles per pair of slabs).
        u32x4 op0[2], op1[2];
        auto widen = [&](u32x4 (&op)[2], const AFrag (&a)[2], const float (&sc2)[2], auto pow2_c) {
            if constexpr (FP8) {
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    uint32_t x0, x1, x2, x3;
                    if constexpr (decltype(pow2_c)::value) {
                        fp8x4_to_bf16x4_pow2(a[pr][0], sc2[pr], x0, x1);
                        fp8x4_to_bf16x4_pow2(a[pr][1], sc2[pr], x2, x3);
                    } else {
                        fp8x4_to_bf16x4(a[pr][0], sc2[pr], x0, x1);
                        fp8x4_to_bf16x4(a[pr][1], sc2[pr], x2, x3);
                    }
                    op[pr] = u32x4{x0, x1, x2, x3};
                }
            } else {
                op[0] = a[0];
                op[1] = a[1];
            }
        };
        auto mfmas = [&](const u32x4 (&op)[2], const u32x4 (&b)[TB]) {
#pragma unroll
            for (int tb = 0; tb < TB; ++tb)
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) acc[pr][tb] = T::mfma32(op[pr], b[tb], acc[pr][tb]);
        };
        // order of a half step: its loads, the LDS reads of the next half step, two products, then the conversions of
        // the next half step spread between the remaining products
        auto order = [&](auto pow2_c, auto loads_c) {
            constexpr int NM = 2 * TB, NV = !FP8 ? 0 : (decltype(pow2_c)::value ? 8 : 34), PER = (NV + NM - 3) / (NM - 2);
            if constexpr (decltype(loads_c)::value) __builtin_amdgcn_sched_group_barrier(0x020, S::NLOAD, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2 + TB, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#pragma unroll
            for (int m = 2; m < NM; ++m) {
                if constexpr (PER > 0) __builtin_amdgcn_sched_group_barrier(0x002, PER, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // slabs past the end are fetched as copies of the last one and never multiplied: the count of loads in flight is
        // the same in every trip.  wait_landed(): all but this wave's loads of the youngest RING - 3 slabs have landed.
        const int last = slab0 + nslab - 1;
        const bool two_chunks = wave + 4 < S::NCH;
        auto wait_landed = [&]() {
            if (two_chunks) wait_vmcnt_le<S::NLOAD * (RING - 3)>();
            else wait_vmcnt_le<(S::NLOAD - 1) * (RING - 3)>();
        };
        // The short road for power-of-two scales is taken by a wave whose block scales are all powers of two (decided
        // once: the two roads are two copies of the loop, so that neither holds a branch between its products).
        bool all_pow2 = false;
        if constexpr (FP8) {
            bool mine = true;
#pragma unroll
            for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine = mine && scale_is_pow2(srow[pr].v[i]);
            all_pow2 = __builtin_amdgcn_ballot_w64(!mine) == 0;
        }
        auto loop = [&](auto pow2_c) {
#pragma unroll
            for (int i = 0; i < RING - 1; ++i) issue(abase, a_voff, B, b_voff, wave, min(slab0 + i, last), i);
            wait_landed();                                       // slabs 0 and 1 of this wave have landed
            bare_barrier();
            float sc[2] = {1.f, 1.f}, scn[2] = {1.f, 1.f};       // block scales of this slab and of the next one
            if constexpr (FP8) {
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) sc[pr] = scn[pr] = scale_at(srow[pr], slab0 >> 2);
            }
            rd(a0, b0, 0, 0);
            widen(op0, a0, sc, pow2_c);
            int cur = 0;
            for (int s = 0; s < nslab; ++s) {
                const int nxt = cur == RING - 1 ? 0 : cur + 1, prv = cur == 0 ? RING - 1 : cur - 1;
                if constexpr (FP8) {
                    if (((slab0 + s + 1) & 3) == 0) {            // a scale block is 128 k = four slabs
#pragma unroll
                        for (int pr = 0; pr < 2; ++pr) scn[pr] = scale_at(srow[pr], (slab0 + s + 1) >> 2);
                    }
                }
                issue(abase, a_voff, B, b_voff, wave, min(slab0 + s + RING - 1, last), prv);
                rd(a1, b1, cur, 1);
                widen(op1, a1, sc, pow2_c);
                mfmas(op0, b0);
                order(pow2_c, std::true_type{});
                rd(a0, b0, nxt, 0);
                widen(op0, a0, scn, pow2_c);
                mfmas(op1, b1);
                order(pow2_c, std::false_type{});
                wait_landed();                                   // this wave's loads of slab s + 2 have landed
                bare_barrier();
                cur = nxt;
                sc[0] = scn[0];
                sc[1] = scn[1];
            }
        };
        if (all_pow2) loop(std::true_type{});
        else loop(std::false_type{});
        __builtin_amdgcn_s_waitcnt(0);                           // nothing may still be writing LDS when the ring is given up
        mfma_settle();
    }
};

}  // namespace mlk
