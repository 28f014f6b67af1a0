// lv_gemm.h — batched prompt evaluation: out[n][m] (+)= sum_k x[n][k] * W[m][k] for n tokens at once, W quantised
// (q4_0 / q8_0), on the matrix cores (reference: the *_batch.comp shader variants selected by
// llava_session.cpp:243-255 when more than one token is pending).
//
// Arithmetic: fp16 MFMA with fp32 accumulation, on operands split in two fp16 halves each.  A dequantised weight
// (q-8)*d or q*d has at most 19 significant bits, an fp32 activation 24: w = wh + wl, x = xh + xl with
// wh = fp16(w), wl = fp16(w - wh) (exact for weights, 2^-22 relative for activations), and
//     x*w ~= xh*wh + xl*wh + xh*wl                      (three MFMAs; the dropped xl*wl term is below 2^-22)
// so the batched path agrees with the one-token fp32 path to fp32 rounding, not to fp16 rounding.
//
// Tiling: workgroup = 256 threads = 4 waves, output tile 128 tokens x 128 weight rows, K step 64 (two quant
// blocks).  One thread dequantises one (row, block) pair per step; every wave owns a 64 x 64 sub-tile = 2 x 2
// v_mfma_f32_32x32x16_f16 tiles.  Global loads of step s+1 are issued before the MFMAs of step s.
#pragma once

#include "lv_kernels.h"

namespace lv {

typedef _Float16 lv_h8 __attribute__((ext_vector_type(8)));
typedef float lv_f16v __attribute__((ext_vector_type(16)));

constexpr int kGemmTile = 128;  // tokens and rows per workgroup
constexpr int kGemmK = 64;      // K per step
constexpr int kGemmLd = kGemmK + 8;  // LDS row stride in halfs (the pad spreads 16-byte reads over the banks)

// x[n][K] fp32 -> xh, xl [n_pad][K] fp16 (rows n..n_pad-1 zero)
__global__ void split_half_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, const float *__restrict__ x, uint32_t n, uint32_t K)
{
    const uint32_t row = blockIdx.y;
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= K) return;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < n) v = *reinterpret_cast<const float4 *>(x + (size_t)row * K + i);
    const float f[4] = {v.x, v.y, v.z, v.w};
    uint16_t h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        h[j] = float_to_half_bits(f[j]);
        l[j] = float_to_half_bits(f[j] - half_bits_to_float(h[j]));
    }
    *reinterpret_cast<uint2 *>(xh + (size_t)row * K + i) = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
    *reinterpret_cast<uint2 *>(xl + (size_t)row * K + i) = make_uint2(l[0] | ((uint32_t)l[1] << 16), l[2] | ((uint32_t)l[3] << 16));
}

// ff[n][F] = a * b / (exp(-b) + 1)   (matmul_silu_ff.comp:96 with a = W3 x, b = W1 x)
__global__ void silu_mul_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, size_t count)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) {
        const float r1 = a[i], r2 = b[i];
        out[i] = r1 * r2 / (__expf(-r2) + 1.f);
    }
}

struct GemmArgs {
    float *out;             // [n][ldo]
    const uint16_t *xh, *xl;  // [n_pad][K] fp16 halves of the activations, n_pad a multiple of 128
    MatView w;              // rows x K
    uint32_t n;             // tokens
    uint32_t ldo;           // floats between output rows
    int accumulate;         // out += instead of out =
};

template <int QT>
__device__ __forceinline__ void gemm_dequant_block(uint16_t *wh, uint16_t *wl, const MatView &w, uint32_t row, uint32_t blk, bool valid,
                                                   const uint4 &c0, const uint4 &c1, uint16_t dbits)
{
    // 32 weights of one block -> 32 hi + 32 lo halfs at wh/wl (contiguous in k)
    const float d = valid ? half_bits_to_float(dbits) : 0.f;
    float v[32];
    if constexpr (QT == 4) {
        const uint32_t q[4] = {c0.x, c0.y, c0.z, c0.w};
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const uint32_t byte = (q[i] >> (8 * b)) & 0xffu;
                v[4 * i + b] = (float)((int)(byte & 15u) - 8) * d;        // element j of the block: low nibble of byte j
                v[16 + 4 * i + b] = (float)((int)(byte >> 4) - 8) * d;    // element j + 16: high nibble
            }
    } else {
        const uint32_t q[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int b = 0; b < 4; b++) v[4 * i + b] = (float)(int)(int8_t)((q[i] >> (8 * b)) & 0xffu) * d;
    }
    (void)w; (void)row; (void)blk;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        uint32_t ph[4], pl[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = v[8 * g + 2 * j], b = v[8 * g + 2 * j + 1];
            const uint16_t ha = float_to_half_bits(a), hb = float_to_half_bits(b);
            const uint16_t la = float_to_half_bits(a - half_bits_to_float(ha)), lb = float_to_half_bits(b - half_bits_to_float(hb));
            ph[j] = ha | ((uint32_t)hb << 16);
            pl[j] = la | ((uint32_t)lb << 16);
        }
        *reinterpret_cast<uint4 *>(wh + 8 * g) = make_uint4(ph[0], ph[1], ph[2], ph[3]);
        *reinterpret_cast<uint4 *>(wl + 8 * g) = make_uint4(pl[0], pl[1], pl[2], pl[3]);
    }
}

template <int QT>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs a)
{
    constexpr int CPB = QT == 4 ? 1 : 2;  // uint4 of codes per block
    __shared__ __attribute__((aligned(16))) uint16_t sXh[kGemmTile * kGemmLd], sXl[kGemmTile * kGemmLd], sWh[kGemmTile * kGemmLd],
        sWl[kGemmTile * kGemmLd];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t tok0 = blockIdx.y * kGemmTile, row0 = blockIdx.x * kGemmTile;
    const uint32_t K = a.w.cols, nb = K / 32, steps = (K + kGemmK - 1) / kGemmK;

    // this thread's weight block of a step: row r_w, block (2*step + b_w)
    const int r_w = tid >> 1, b_w = tid & 1;
    const uint32_t wrow = row0 + r_w;
    const bool wrow_ok = wrow < a.w.rows;
    // this thread's four 16-byte pieces of the activation tile of a step: token rows tid/8 + 32*i, halfs (tid%8)*8..+7
    const int xr = tid >> 3, xc = (tid & 7) * 8;

    uint4 c0 = make_uint4(0, 0, 0, 0), c1 = c0;
    uint16_t dbits = 0;
    bool wvalid = false;
    uint4 gh[4], gl[4];
    auto fetch = [&](uint32_t step) {
        const uint32_t blk = 2 * step + b_w;
        wvalid = wrow_ok && blk < nb;
        const size_t sb = (size_t)(wvalid ? wrow : 0) * nb + (wvalid ? blk : 0);
        c0 = a.w.codes[sb * CPB];
        if constexpr (QT == 8) c1 = a.w.codes[sb * CPB + 1];
        dbits = a.w.scales[sb];
        const uint32_t k = step * kGemmK + xc;
        const bool kok = k < K;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const size_t off = (size_t)(tok0 + xr + 32 * i) * K + (kok ? k : 0);
            gh[i] = *reinterpret_cast<const uint4 *>(a.xh + off);
            gl[i] = *reinterpret_cast<const uint4 *>(a.xl + off);
            if (!kok) gh[i] = gl[i] = make_uint4(0, 0, 0, 0);
        }
    };

    lv_f16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    fetch(0);
    for (uint32_t step = 0; step < steps; step++) {
        // registers -> LDS
        gemm_dequant_block<QT>(sWh + r_w * kGemmLd + b_w * 32, sWl + r_w * kGemmLd + b_w * 32, a.w, wrow, 0, wvalid, c0, c1, dbits);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<uint4 *>(sXh + (xr + 32 * i) * kGemmLd + xc) = gh[i];
            *reinterpret_cast<uint4 *>(sXl + (xr + 32 * i) * kGemmLd + xc) = gl[i];
        }
        __syncthreads();
        if (step + 1 < steps) fetch(step + 1);
#pragma unroll
        for (int kk = 0; kk < kGemmK / 16; kk++) {
            const int ko = kk * 16 + (lane >> 5) * 8;
            lv_h8 xh[2], xl[2], wh[2], wl[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int xrow = wm * 64 + t * 32 + (lane & 31), wr = wn * 64 + t * 32 + (lane & 31);
                xh[t] = *reinterpret_cast<const lv_h8 *>(sXh + xrow * kGemmLd + ko);
                xl[t] = *reinterpret_cast<const lv_h8 *>(sXl + xrow * kGemmLd + ko);
                wh[t] = *reinterpret_cast<const lv_h8 *>(sWh + wr * kGemmLd + ko);
                wl[t] = *reinterpret_cast<const lv_h8 *>(sWl + wr * kGemmLd + ko);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl[i], wh[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh[i], wl[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh[i], wh[j], acc[i][j], 0, 0, 0);
                }
        }
        __syncthreads();
    }

    // D[i][j]: i = token within the 32-tile, j = weight row; lane l holds j = l%32 and, in register r,
    // i = 8*(r/4) + 4*(l/32) + r%4
#pragma unroll
    for (int ti = 0; ti < 2; ti++)
#pragma unroll
        for (int tj = 0; tj < 2; tj++) {
            const uint32_t m = row0 + wn * 64 + tj * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t n = tok0 + wm * 64 + ti * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (n < a.n && m < a.w.rows) {
                    float *dst = a.out + (size_t)n * a.ldo + m;
                    *dst = a.accumulate ? *dst + acc[ti][tj][r] : acc[ti][tj][r];
                }
            }
        }
}

}  // namespace lv
