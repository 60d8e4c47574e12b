// 128-point Sylvester Hadamard on one wavefront, two elements per lane.
//
// Butterfly order is fixed (stage h = 1, 2, 4 .. 64; element i with i & h == 0 gets
// a + b, element i + h gets a - b, a the lower element), in fp32, so that the
// rotated activation rounds to the same fp16 bits on every implementation that
// follows the same order.  Scale 1/sqrt(128) as in
// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:44-46.
//
// Cross-lane exchange stays in the vector ALU: DPP moves for lane distances 1, 2,
// 4, 8 and the gfx950 row-swap instructions for 16 and 32; no LDS round trips.
#pragma once

#include <hip/hip_runtime.h>

namespace berth {

template <int CTRL, int BANK_MASK = 0xF>
__device__ __forceinline__ float dpp_mov(float old, float src)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                                 __builtin_bit_cast(int, src), CTRL, 0xF,
                                                                 BANK_MASK, false));
}

// value of lane (lane ^ D) for D in {1, 2, 4, 8}
template <int D>
__device__ __forceinline__ float lane_xor_dpp(float v)
{
    if constexpr (D == 1) return dpp_mov<0xB1>(v, v);                  // quad_perm [1,0,3,2]
    else if constexpr (D == 2) return dpp_mov<0x4E>(v, v);             // quad_perm [2,3,0,1]
    else if constexpr (D == 4) {
        float p = dpp_mov<0x104, 0x5>(v, v);                           // row_shl:4 into lanes with bit 2 clear
        return dpp_mov<0x114, 0xA>(p, v);                              // row_shr:4 into lanes with bit 2 set
    } else return dpp_mov<0x128>(v, v);                                // row_ror:8
}

// one butterfly stage over lane distance D < 16: lower lane a + b, upper lane a - b.
// sgn is +1 in the lower lane and -1 in the upper lane of the pair, so both are
// fma(own, sgn, partner) with a single rounding: a + b and (a) - (b) exactly.
template <int D>
__device__ __forceinline__ float had_stage_dpp(float v, float sgn)
{
    return __builtin_fmaf(v, sgn, lane_xor_dpp<D>(v));
}

// stages over lane distance 16 and 32.  v_permlane16_swap_b32 a, b exchanges the
// odd 16-lane rows of a with the even rows of b; with a = b = v on entry, a ends up
// holding the lower element (lo) and b the upper element (hi) of every lane's pair,
// and the butterfly is lo + sgn * hi.  v_permlane32_swap_b32 does the same for the
// two 32-lane halves.  Written as inline assembly (two read-write registers); the
// s_nop pads cover the data hazards the compiler cannot see around inline code.
__device__ __forceinline__ float had_stage_swap16(float v, float sgn)
{
    float lo = v, hi = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return __builtin_fmaf(hi, sgn, lo);
}

__device__ __forceinline__ float had_stage_swap32(float v, float sgn)
{
    float lo = v, hi = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return __builtin_fmaf(hi, sgn, lo);
}

// value of lane (lane ^ 16) / (lane ^ 32): after the swap one of the two registers
// holds the partner's value in every lane (the lower rows find it in hi, the upper
// rows in lo)
__device__ __forceinline__ float lane_xor_swap16(float v)
{
    float lo = v, hi = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return (__lane_id() & 16) ? lo : hi;
}

__device__ __forceinline__ float lane_xor_swap32(float v)
{
    float lo = v, hi = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return (__lane_id() & 32) ? lo : hi;
}

// lane l holds elements 2l (v0) and 2l+1 (v1) of a 128 vector
__device__ __forceinline__ void had128_wave(float& v0, float& v1, int lane)
{
    const float a = v0, b = v1;
    v0 = a + b;
    v1 = a - b;
    const float s1 = (lane & 1) ? -1.0f : 1.0f;
    const float s2 = (lane & 2) ? -1.0f : 1.0f;
    const float s4 = (lane & 4) ? -1.0f : 1.0f;
    const float s8 = (lane & 8) ? -1.0f : 1.0f;
    const float s16 = (lane & 16) ? -1.0f : 1.0f;
    const float s32 = (lane & 32) ? -1.0f : 1.0f;
    v0 = had_stage_dpp<1>(v0, s1);   v1 = had_stage_dpp<1>(v1, s1);
    v0 = had_stage_dpp<2>(v0, s2);   v1 = had_stage_dpp<2>(v1, s2);
    v0 = had_stage_dpp<4>(v0, s4);   v1 = had_stage_dpp<4>(v1, s4);
    v0 = had_stage_dpp<8>(v0, s8);   v1 = had_stage_dpp<8>(v1, s8);
    // distance 16 and 32: lower rows hold lo, upper rows hold hi of each pair, so
    // the result is lo + hi in the lower lane and lo - hi in the upper lane
    v0 = had_stage_swap16(v0, s16);  v1 = had_stage_swap16(v1, s16);
    v0 = had_stage_swap32(v0, s32);  v1 = had_stage_swap32(v1, s32);
}

// 128-point Hadamard with eight consecutive elements per lane and sixteen lanes
// (one DPP row) per vector, so a wave rotates four vectors at once: stages 1, 2, 4
// stay inside the lane, stages 8 .. 64 are DPP exchanges inside the row.  Same
// butterfly order and the same exact sums as had128_wave.
__device__ __forceinline__ void had128_row16(float (&v)[8], int lane)
{
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((i & h) == 0) {
                const float a = v[i], b = v[i + h];
                v[i] = a + b;
                v[i + h] = a - b;
            }
        }
    }
    const float s1 = (lane & 1) ? -1.0f : 1.0f;
    const float s2 = (lane & 2) ? -1.0f : 1.0f;
    const float s4 = (lane & 4) ? -1.0f : 1.0f;
    const float s8 = (lane & 8) ? -1.0f : 1.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = had_stage_dpp<1>(v[i], s1);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = had_stage_dpp<2>(v[i], s2);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = had_stage_dpp<4>(v[i], s4);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = had_stage_dpp<8>(v[i], s8);
}

}  // namespace berth
