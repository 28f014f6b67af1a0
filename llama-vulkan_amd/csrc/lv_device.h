// lv_device.h — wave64 building blocks shared by every kernel: DPP reductions, fp16 and code unpacking.
// gfx950 only (64-wide wavefronts, DPP row operations).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

// The kernels lean on gfx950 behaviour the HIP memory model does not promise (write-through stores acknowledged once every
// XCD can see them, non-temporal loads that pass the CU's cache, the XCC id register): no other device target is built.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "llama-vulkan_amd device code is written for gfx950 (MI355X) only"
#endif

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
// Four per-lane partials (one per matrix row) -> every lane of 16-lane row j holds the total of partial
// kRowOfLaneGroup[j]: two v_permlane32_swap + one v_permlane16_swap fold the 64 lanes down to 16 per partial,
// then DPP adds finish inside the rows.
__device__ __forceinline__ float quad_partials_sum(float p0, float p1, float p2, float p3)
{
    // swap32(a, b): a' = [a.lo32 | b.lo32], b' = [a.hi32 | b.hi32]
    auto s01 = __builtin_amdgcn_permlane32_swap(__float_as_uint(p0), __float_as_uint(p1), false, false);
    auto s23 = __builtin_amdgcn_permlane32_swap(__float_as_uint(p2), __float_as_uint(p3), false, false);
    const float a = __uint_as_float(s01[0]) + __uint_as_float(s01[1]);  // lanes 0-31: p0 pairs, 32-63: p1 pairs
    const float b = __uint_as_float(s23[0]) + __uint_as_float(s23[1]);  // lanes 0-31: p2 pairs, 32-63: p3 pairs
    // swap16(a, b): a' = [a.r0 b.r0 a.r2 b.r2], b' = [a.r1 b.r1 a.r3 b.r3]
    auto t = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    const float c = __uint_as_float(t[0]) + __uint_as_float(t[1]);      // rows of 16 lanes hold p0, p2, p1, p3
    return group16_sum(c);
}
// The same for partials whose lanes 0-31 and 32-63 belong to two different matrix rows (tiles that carry 32 blocks of each
// of two rows): eight totals.  In s01 the 16-lane rows hold the totals of [p0 lower half, p0 upper half, p1 lower, p1 upper],
// in s23 those of p2 and p3.
__device__ __forceinline__ void quad_partials_sum_halves(float p0, float p1, float p2, float p3, float &s01, float &s23)
{
    auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(p0), __float_as_uint(p1), false, false);  // [p0.lo | p1.lo], [p0.hi | p1.hi]
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(p2), __float_as_uint(p3), false, false);
    auto ta = __builtin_amdgcn_permlane16_swap(a[0], a[1], false, false);   // [lo.r0 hi.r0 lo.r2 hi.r2], [lo.r1 hi.r1 lo.r3 hi.r3]
    auto tb = __builtin_amdgcn_permlane16_swap(b[0], b[1], false, false);
    s01 = group16_sum(__uint_as_float(ta[0]) + __uint_as_float(ta[1]));
    s23 = group16_sum(__uint_as_float(tb[0]) + __uint_as_float(tb[1]));
}
// which of the four partials ends up in 16-lane row j of the result above
__device__ __forceinline__ int quad_partial_of_lane(int lane)
{
    const int j = lane >> 4;
    return ((j & 1) << 1) | (j >> 1);
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
//
// Nibble -> float without a per-element extract: a byte 0x0q read as an OCP fp8 E4M3 number is exactly
// q * 2^-9 for every q in 0..15 (q < 8 are the subnormals m * 2^-9, q >= 8 have exponent field 1 and value
// (8 + m) * 2^-9).  v_cvt_pk_f32_fp8 converts two such bytes per instruction, so eight codes cost two masks,
// one shift and four converts.  The factor 2^9 is applied once per block (exact).
typedef float lv_float2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float q4_block_dot(const uint4 &q, const float (&x)[32])
{
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = w[i] & 0x0f0f0f0fu;
        const uint32_t hi = (w[i] >> 4) & 0x0f0f0f0fu;
        const lv_float2 l01 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false), l23 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
        const lv_float2 h01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false), h23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
        acc = fmaf(l01.x, x[4 * i + 0], acc);
        acc = fmaf(l01.y, x[4 * i + 1], acc);
        acc = fmaf(l23.x, x[4 * i + 2], acc);
        acc = fmaf(l23.y, x[4 * i + 3], acc);
        acc = fmaf(h01.x, x[16 + 4 * i + 0], acc);
        acc = fmaf(h01.y, x[16 + 4 * i + 1], acc);
        acc = fmaf(h23.x, x[16 + 4 * i + 2], acc);
        acc = fmaf(h23.y, x[16 + 4 * i + 3], acc);
    }
    return acc * 512.f;
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
