// lv_device.h — wave64 building blocks shared by every kernel: DPP reductions, fp16 and code unpacking.
// gfx950 only (64-wide wavefronts, DPP row operations).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lv {

constexpr int kWave = 64;

// ---- DPP cross-lane moves --------------------------------------------------------------------------------
// dpp_ctrl encodings: quad_perm = 8 bits of 2-bit lane selectors; 0x140 row_mirror; 0x141 row_half_mirror.
template <int Ctrl>
__device__ __forceinline__ float dpp_mov(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xf, 0xf, true));
}

// sum over the 4 / 8 / 16 consecutive lanes this lane belongs to; every lane of the group gets the total
__device__ __forceinline__ float group4_sum(float v)
{
    v += dpp_mov<0xB1>(v);  // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);  // quad_perm [2,3,0,1]
    return v;
}
__device__ __forceinline__ float group8_sum(float v)
{
    v = group4_sum(v);
    v += dpp_mov<0x141>(v);  // row_half_mirror: lane i <- lane 7-i of its half row
    return v;
}
__device__ __forceinline__ float group16_sum(float v)
{
    v = group8_sum(v);
    v += dpp_mov<0x140>(v);  // row_mirror: lane i <- lane 15-i of its row
    return v;
}
// whole wavefront; every lane gets the total
__device__ __forceinline__ float wave_sum(float v)
{
    v = group16_sum(v);
    v += __shfl_xor(v, 16, kWave);
    v += __shfl_xor(v, 32, kWave);
    return v;
}
template <int Lanes>
__device__ __forceinline__ float group_sum(float v)
{
    static_assert(Lanes == 4 || Lanes == 8 || Lanes == 16 || Lanes == 64, "group size");
    if constexpr (Lanes == 4) return group4_sum(v);
    else if constexpr (Lanes == 8) return group8_sum(v);
    else if constexpr (Lanes == 16) return group16_sum(v);
    else return wave_sum(v);
}

// ---- fp16 ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float half_bits_to_float(uint16_t h)
{
    return __half2float(__ushort_as_half(h));  // v_cvt_f32_f16: exact, subnormals included
}
__device__ __forceinline__ uint16_t float_to_half_bits(float f)
{
    return __half_as_ushort(__float2half_rn(f));  // v_cvt_f16_f32, round to nearest even
}

// ---- code unpacking --------------------------------------------------------------------------------------
// byte k of a dword as float (v_cvt_f32_ubyteK)
template <int K>
__device__ __forceinline__ float ubyte_to_float(uint32_t v)
{
    return (float)((v >> (8 * K)) & 0xffu);
}

// Sum over one q4_0 block of code*x with the codes left unsigned (0..15); the caller subtracts 8*sum(x).
// GGML order (llava_buffer.cpp:361-369): byte j holds element j in its low nibble, element j+16 in its high one.
__device__ __forceinline__ float q4_block_dot(const uint4 &q, const float (&x)[32])
{
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = w[i] & 0x0f0f0f0fu;
        const uint32_t hi = (w[i] >> 4) & 0x0f0f0f0fu;
        acc = fmaf(ubyte_to_float<0>(lo), x[4 * i + 0], acc);
        acc = fmaf(ubyte_to_float<1>(lo), x[4 * i + 1], acc);
        acc = fmaf(ubyte_to_float<2>(lo), x[4 * i + 2], acc);
        acc = fmaf(ubyte_to_float<3>(lo), x[4 * i + 3], acc);
        acc = fmaf(ubyte_to_float<0>(hi), x[16 + 4 * i + 0], acc);
        acc = fmaf(ubyte_to_float<1>(hi), x[16 + 4 * i + 1], acc);
        acc = fmaf(ubyte_to_float<2>(hi), x[16 + 4 * i + 2], acc);
        acc = fmaf(ubyte_to_float<3>(hi), x[16 + 4 * i + 3], acc);
    }
    return acc;
}

// Sum over one q8_0 block of (code+128)*x: codes are biased to unsigned by flipping the sign bit so the byte
// converts apply; the caller subtracts 128*sum(x).
__device__ __forceinline__ float q8_block_dot(const uint4 &qa, const uint4 &qb, const float (&x)[32])
{
    const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t u = w[i] ^ 0x80808080u;
        acc = fmaf(ubyte_to_float<0>(u), x[4 * i + 0], acc);
        acc = fmaf(ubyte_to_float<1>(u), x[4 * i + 1], acc);
        acc = fmaf(ubyte_to_float<2>(u), x[4 * i + 2], acc);
        acc = fmaf(ubyte_to_float<3>(u), x[4 * i + 3], acc);
    }
    return acc;
}

}  // namespace lv
