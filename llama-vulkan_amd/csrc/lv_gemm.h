// lv_gemm.h — batched prompt evaluation: out[n][m] (+)= sum_k x[n][k] * W[m][k] for n tokens at once, W quantised
// (q4_0 / q8_0), on the matrix cores (reference: the *_batch.comp shader variants selected by
// llava_session.cpp:243-255 when more than one token is pending).
//
// Arithmetic: fp16 MFMA with fp32 accumulation, in the order of the reference's shaders (matmul.glsl:41-74: the block
// dot on the integer codes first, then times the block's scale, then added to the running sum).  A code (q-8 or q) is
// a small integer, exact in fp16; an fp32 activation is split in two fp16 halves, x = xh + xl (2^-22 relative):
//     sum_k x[k]*code[k] = sum_k xh[k]*code[k] + sum_k xl[k]*code[k]      (two MFMAs per 16 k, every product exact)
// per block of 32 k into a scratch accumulator, which is then multiplied by the block's scale d[row] (one scale per
// lane: in the MFMA result a lane holds one weight row) and added to the fp32 result.  The batched path therefore
// agrees with the one-token fp32 path to fp32 rounding, not to fp16 rounding.
//
// Operands in memory.  The kernel's inner loop does nothing but MFMAs and the scale multiply-adds: the codes are not
// unpacked there.  A model keeps a second copy of its layer matrices for this path only (the "prompt copy", made when the
// first batch is evaluated): every code as the fp16 integer it stands for, and the block scales as fp32, both in the
// order in which a workgroup's tile lies in LDS.  The producers of the activations (the split, norm and SwiGLU kernels
// below) write the two halves in tile order as well.  With that a K step of a tile is one contiguous run of memory,
// which global_load_lds_dwordx4 copies to LDS without passing through registers, four steps ahead of the MFMAs.
//   weights      [row tile of 256][K/8 chunks][256 rows][8 halfs]
//   scales       [row tile of 256][K/32 blocks][256 rows] fp32
//   activations  [token tile of 128][K/8 chunks][128 tokens][8 halfs], high halves and low halves apart
// K is padded to a multiple of 64 with zero codes and zero activations, rows to 256 with zero scales.
// In LDS a chunk row of 16 bytes is what one lane feeds an MFMA (v_mfma_f32_32x32x16_f16: lane l holds row l%32,
// k (l/32)*8..+7), and 32 consecutive lanes read 512 consecutive bytes: no bank conflicts, no padding.
//
// Tiling: workgroup = 8 waves, output tile 128 tokens x 256 weight rows, K step 32 (one quant block), every wave a
// 64 x 64 sub-tile (2 x 2 MFMA tiles).  Four LDS stages of 33 KB.
#pragma once

#include "lv_kernels.h"

namespace lv {

typedef _Float16 lv_h8 __attribute__((ext_vector_type(8)));
typedef float lv_f16v __attribute__((ext_vector_type(16)));
typedef float lv_f4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lv_lds_void;
typedef const __attribute__((address_space(1))) void lv_glb_void;

constexpr int kGemmTile = 128;   // tokens per workgroup (batches are padded to multiples of it)
constexpr int kGemmRows = 256;   // weight rows per workgroup (the prompt copy pads matrices to multiples of it)
constexpr int kGemmK = 64;       // K is padded to multiples of it; the unit in which K is cut in slices
constexpr int kGemmStep = 32;    // K per pipeline stage: one quant block
constexpr int kGemmStages = 4;
constexpr int kGemmWBytes = kGemmStep / 8 * kGemmRows * 16;                    // 16 KB of weights per stage
constexpr int kGemmXBytes = kGemmStep / 8 * kGemmTile * 16;                    // 8 KB per activation half
constexpr int kGemmScBytes = kGemmRows * 4;
constexpr int kGemmStageBytes = kGemmWBytes + 2 * kGemmXBytes + kGemmScBytes;  // 33 KB
constexpr int kGemmLdsBytes = kGemmStages * kGemmStageBytes;                   // 132 KB: one workgroup per CU

__host__ __device__ constexpr uint32_t gemm_k_padded(uint32_t K) { return (K + kGemmK - 1) / kGemmK * kGemmK; }
__host__ __device__ constexpr uint32_t gemm_rows_padded(uint32_t rows) { return (rows + kGemmRows - 1) / kGemmRows * kGemmRows; }
// halfs (2-byte units) of a matrix's prompt copy: the codes, then the scale plane
__host__ __device__ constexpr uint64_t gemm_copy_code_halfs(uint32_t rows, uint32_t K) { return (uint64_t)gemm_rows_padded(rows) * gemm_k_padded(K); }
__host__ __device__ constexpr uint64_t gemm_copy_halfs(uint32_t rows, uint32_t K)
{
    return gemm_copy_code_halfs(rows, K) + (uint64_t)gemm_rows_padded(rows) * (gemm_k_padded(K) / 32) * 2;
}
// offset in halfs of the 8 halfs (token, k..k+7), k a multiple of 8, in a tile-ordered activation plane of padded width Kp
__device__ __forceinline__ size_t gemm_x_offset(uint32_t token, uint32_t k, uint32_t Kp)
{
    return (((size_t)(token / kGemmTile) * (Kp / 8) + k / 8) * kGemmTile + token % kGemmTile) * 8;
}

__device__ __forceinline__ void gemm_split8(uint4 &h, uint4 &l, const float (&f)[8])
{
    uint32_t hw[4], lw[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint16_t h0 = float_to_half_bits(f[2 * j]), h1 = float_to_half_bits(f[2 * j + 1]);
        const uint16_t l0 = float_to_half_bits(f[2 * j] - half_bits_to_float(h0)), l1 = float_to_half_bits(f[2 * j + 1] - half_bits_to_float(h1));
        hw[j] = (uint32_t)h0 | ((uint32_t)h1 << 16);
        lw[j] = (uint32_t)l0 | ((uint32_t)l1 << 16);
    }
    h = make_uint4(hw[0], hw[1], hw[2], hw[3]);
    l = make_uint4(lw[0], lw[1], lw[2], lw[3]);
}

// The producers of activation halves work a token row at a time: one 256-thread workgroup per row of the padded batch.
// Workgroups are dealt to the 8 XCDs in turn; the row a workgroup takes is chosen so that the 8 tokens whose 16-byte chunks
// share a 128-byte line are written through one XCD's L2.
__device__ __forceinline__ uint32_t gemm_producer_row(uint32_t b) { return (b >> 6) * 64 + (b & 7) * 8 + ((b >> 3) & 7); }   // n_pad is a multiple of 128

// The halves are written for 2^S * x, S chosen per row so that the largest element lies in [2^14, 2^15): the low half of an
// element then stays a normal fp16 number down to 2^-14 of the row's largest (unscaled, the low half of anything below
// 0.125 is a subnormal and the pair carries an absolute error of 2^-25), and a row cannot overflow fp16 whatever its
// size.  xscale[row] = 2^-S, which the GEMM multiplies into its result: powers of two, nothing is rounded.
// Returns 2^S for a row whose largest magnitude is `big`; *down = 2^-S.  1 for an all-zero or non-finite row.
__device__ __forceinline__ float gemm_row_scale(float big, float *down)
{
    const int eb = (int)((__float_as_uint(big) >> 23) & 0xffu);
    const int S = (eb == 0 || eb == 255) ? 0 : max(-100, min(100, 14 - (eb - 127)));
    *down = __uint_as_float((uint32_t)(127 - S) << 23);
    return __uint_as_float((uint32_t)(127 + S) << 23);
}

// One row of activations -> its two halves and its scale.  value(f, i) yields the 8 elements of chunk i (i < K / 8).
// PER > 0: the row (at most 256 * 8 * PER elements) is evaluated once and kept in registers; PER = 0: any length, evaluated
// twice (largest magnitude first, then the halves; the second pass finds its inputs in L2).
template <int PER, class Value>
__device__ __forceinline__ void gemm_write_row(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, float *__restrict__ xscale, uint32_t row, bool live,
                                               uint32_t K, uint32_t Kp, float *lds, Value value)
{
    const uint32_t n8 = K / 8, chunks = Kp / 8;
    float big = 0.f;
    float keep[PER > 0 ? PER : 1][8];
    if constexpr (PER > 0) {
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const uint32_t i = threadIdx.x + j * 256;
#pragma unroll
            for (int e = 0; e < 8; e++) keep[j][e] = 0.f;
            if (live && i < n8) value(keep[j], i);
#pragma unroll
            for (int e = 0; e < 8; e++) big = fmaxf(big, fabsf(keep[j][e]));
        }
    } else {
        if (live)
            for (uint32_t i = threadIdx.x; i < n8; i += 256) {
                float f[8];
                value(f, i);
#pragma unroll
                for (int e = 0; e < 8; e++) big = fmaxf(big, fabsf(f[e]));
            }
    }
    big = block_max_256(big, lds);
    float down;
    const float up = gemm_row_scale(big, &down);
    if (threadIdx.x == 0) xscale[row] = down;
    auto put = [&](uint32_t i, const float (&f)[8]) {
        float g[8];
#pragma unroll
        for (int e = 0; e < 8; e++) g[e] = f[e] * up;
        uint4 h, l;
        gemm_split8(h, l, g);
        const size_t o = gemm_x_offset(row, i * 8, Kp);
        *reinterpret_cast<uint4 *>(xh + o) = h;
        *reinterpret_cast<uint4 *>(xl + o) = l;
    };
    if constexpr (PER > 0) {
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const uint32_t i = threadIdx.x + j * 256;
            if (i < chunks) put(i, keep[j]);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < chunks; i += 256) {
            float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (live && i < n8) value(f, i);
            put(i, f);
        }
    }
}

// x[n][K] fp32 -> xh, xl (tile order, n_pad tokens x Kp; everything outside n x K is written as zero), xscale[n_pad].
// K a multiple of 8; with PER > 0, Kp <= 2048 * PER.  For inputs of unknown size (lv_kernel_gemm's activations).
template <int PER>
__global__ __launch_bounds__(256) void split_rows_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, float *__restrict__ xscale,
                                                          const float *__restrict__ x, uint32_t n, uint32_t K, uint32_t Kp)
{
    __shared__ float lds[4];
    const uint32_t row = gemm_producer_row(blockIdx.x);
    const bool live = row < n;
    const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)(live ? row : 0) * K);
    gemm_write_row<PER>(xh, xl, xscale, row, live, K, Kp, lds, [&](float (&f)[8], uint32_t i) {
        const float4 a = src[2 * i], b = src[2 * i + 1];
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    });
}

// The two elementwise producers inside a prompt batch write unscaled halves (no xscale): attention outputs and SwiGLU
// products are of the size of their rows' largest elements often enough that the 2^-25 absolute error of an unscaled pair is
// of the order of fp32 rounding, and a pass over the row for its maximum costs more than it gains (measured: the same
// logit errors, the prompt 3 % slower, because a row at a time means 16-byte writes 2 KB apart).
// Thread -> (token, chunk of 8 k): a wave covers 8 tokens x 8 chunks, so that it reads 256 consecutive bytes of each
// token's fp32 row and writes, per chunk, the 128 consecutive bytes of its 8 tokens.  grid (Kp / 64, n_pad / 32), 256 threads.
__device__ __forceinline__ void gemm_producer_coords(uint32_t &token, uint32_t &k)
{
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    token = blockIdx.y * 32 + wave * 8 + (lane >> 3);
    k = blockIdx.x * 64 + (lane & 7) * 8;
}

// x[n][K] fp32 -> xh, xl (tile order, n_pad tokens x Kp; everything outside n x K is written as zero)
__global__ __launch_bounds__(256) void split_half_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, const float *__restrict__ x, uint32_t n,
                                                          uint32_t K, uint32_t Kp)
{
    uint32_t token, k;
    gemm_producer_coords(token, k);
    if (k >= Kp) return;
    float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (token < n && k < K) {       // K is a multiple of 8: a chunk lies inside or outside
        const float4 a = *reinterpret_cast<const float4 *>(x + (size_t)token * K + k), b = *reinterpret_cast<const float4 *>(x + (size_t)token * K + k + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
    uint4 h, l;
    gemm_split8(h, l, f);
    const size_t o = gemm_x_offset(token, k, Kp);
    *reinterpret_cast<uint4 *>(xh + o) = h;
    *reinterpret_cast<uint4 *>(xl + o) = l;
}

// ff[n][F] = a * b / (exp(-b) + 1) (matmul_silu_ff.comp:96 with a = W3 x, b = W1 x), written as the two fp16 halves
// the down projection's GEMM reads (the fp32 product is never stored); layout and grid of split_half_kernel
__global__ __launch_bounds__(256) void silu_split_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, const float *__restrict__ a,
                                                          const float *__restrict__ b, uint32_t n, uint32_t K, uint32_t Kp)
{
    uint32_t token, k;
    gemm_producer_coords(token, k);
    if (k >= Kp) return;
    float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (token < n && k < K) {
        const float *pa = a + (size_t)token * K + k, *pb = b + (size_t)token * K + k;
        const float4 a0 = *reinterpret_cast<const float4 *>(pa), a1 = *reinterpret_cast<const float4 *>(pa + 4);
        const float4 b0 = *reinterpret_cast<const float4 *>(pb), b1 = *reinterpret_cast<const float4 *>(pb + 4);
        const float av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w}, bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = av[j] * bv[j] / (__expf(-bv[j]) + 1.f);
    }
    uint4 h, l;
    gemm_split8(h, l, f);
    const size_t o = gemm_x_offset(token, k, Kp);
    *reinterpret_cast<uint4 *>(xh + o) = h;
    *reinterpret_cast<uint4 *>(xl + o) = l;
}

constexpr int kGemmMaxMats = 4;

// SwiGLU for the feed-forward rows f0 .. F-1 whose gate and up products come from a K-sliced launch over the last row tiles
// of a pair copy (expand_codes_kernel<.., true>): parts[s][token][tail_rows] hold slice s in the pair copy's row order
// (32 gate rows, then the same 32 up rows), summed slice 0 first.  Output as silu_split_kernel's, at columns f0 .. of the
// activation tile.  f0 and F are multiples of 128.  grid ((F - f0) / 64, n_pad / 32), 256 threads.
struct SiluTailArgs {
    uint16_t *fh, *fl;
    const float *parts[kGemmMaxMats];
    uint32_t nparts, n, F, Fp, f0, tail_rows;
};
__global__ __launch_bounds__(256) void silu_pair_tail_kernel(SiluTailArgs a)
{
    uint32_t token, k;
    gemm_producer_coords(token, k);                 // k counts from f0
    const uint32_t f = a.f0 + k;
    if (f >= a.F) return;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (token < a.n) {
        const uint32_t prow = k / 128 * 256 + (k % 128) / 32 * 64 + k % 32;     // the chunk's 8 gate rows; their up rows follow 32 further on
        float g[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, u[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (uint32_t s = 0; s < a.nparts; s++) {
            const float *p = a.parts[s] + (size_t)token * a.tail_rows + prow;
            const float4 g0 = *reinterpret_cast<const float4 *>(p), g1 = *reinterpret_cast<const float4 *>(p + 4);
            const float4 u0 = *reinterpret_cast<const float4 *>(p + 32), u1 = *reinterpret_cast<const float4 *>(p + 36);
            g[0] += g0.x; g[1] += g0.y; g[2] += g0.z; g[3] += g0.w; g[4] += g1.x; g[5] += g1.y; g[6] += g1.z; g[7] += g1.w;
            u[0] += u0.x; u[1] += u0.y; u[2] += u0.z; u[3] += u0.w; u[4] += u1.x; u[5] += u1.y; u[6] += u1.z; u[7] += u1.w;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = g[j] * u[j] / (__expf(-u[j]) + 1.f);
    }
    uint4 h, l;
    gemm_split8(h, l, v);
    const size_t o = gemm_x_offset(token, f, a.Fp);
    *reinterpret_cast<uint4 *>(a.fh + o) = h;
    *reinterpret_cast<uint4 *>(a.fl + o) = l;
}

struct GemmArgs {
    // up to four matrices of one shape applied to the same activations in one launch: q, k and v of a layer together fill the CUs that each alone leaves idle
    float *outs[kGemmMaxMats];          // [n][ldo] each
    const uint16_t *xh, *xl;            // activation halves, tile order, n_pad x Kp
    const uint16_t *w16[kGemmMaxMats];  // prompt copies (codes, then scales)
    uint32_t rows, K;                   // of every matrix
    uint32_t n;                         // tokens
    uint32_t ldo;                       // floats between output rows
    int accumulate;                     // out += instead of out =
    const float *xscale;                // null, or [n_pad]: the activation halves of token t stand for x / xscale[t] (a power of two)
    // 0: nz matrices.  Otherwise the launch splits K: w16[] all name one matrix, slice y multiplies the
    // K range y*slice_k .. (y+1)*slice_k-1 (slice_k a multiple of 64) into outs[y], and gemm_reduce_kernel adds the slices
    // up (a matrix with few rows and a long K, like the down projection, fills the CUs that way)
    uint32_t slice_k;
    uint32_t nz;                        // matrices or slices in this launch
    // gemm_kernel<true> only: w16[0] is a PAIR copy (expand_codes_kernel) of rows / 2 gate and rows / 2 up rows, and the
    // result is not the products but ff = gate * up / (exp(-up) + 1) (matmul_silu_ff.comp:96) as the two fp16 halves the
    // down projection's GEMM reads: tile order, n_pad x fKp
    uint16_t *fh, *fl;
    uint32_t fKp;
    // gemm_rows16_kernel only: for a matrix z with half_out[z] set the result is stored as fp16 (round to nearest even, what
    // copy_to_cache.comp:29-37 does to K and V) at half_out[z][(*row_ptr + row_add + token) * ldo + m], rows below row_limit:
    // the k and v products of a prompt batch go straight into their cache rows
    uint16_t *half_out[kGemmMaxMats];
    const uint32_t *row_ptr;
    uint32_t row_add, row_limit;
    // a launch over part of the row tiles: tile_count of them (0: all) from tile0 on; fp32 results then go to column
    // m - tile0 * 256 of their output rows
    uint32_t tile0, tile_count;
};

// out[n][ldo] (+)= p[0] + p[1] (+ p[2] + p[3]), the K slices of one product, each [n][rows]; always summed in this order
struct GemmReduceArgs {
    float *out;
    const float *parts[kGemmMaxMats];
    uint32_t nparts, rows, ldo, n;
    int accumulate;
};
__global__ void gemm_reduce_kernel(GemmReduceArgs a)
{
    const uint32_t row = blockIdx.y, c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c >= a.rows) return;
    const size_t src = (size_t)row * a.rows + c;
    float4 s = *reinterpret_cast<const float4 *>(a.parts[0] + src);
    for (uint32_t i = 1; i < a.nparts; i++) {
        const float4 v = *reinterpret_cast<const float4 *>(a.parts[i] + src);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    float4 *dst = reinterpret_cast<float4 *>(a.out + (size_t)row * a.ldo + c);
    if (a.accumulate) {
        const float4 o = *dst;
        s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
    }
    *dst = s;
}

// The prompt copy of one matrix: codes as fp16 integers (q4_0: q - 8, q8_0: q) and scales as fp32, in the tile order
// described at the top of this file.  One thread per (row of the padded matrix, block of the padded K); consecutive
// threads take consecutive rows, so that every 16-byte chunk row they write is next to its neighbour's.
// PAIR: the copy of the feed-forward's two input matrices as ONE matrix of 2 x rows whose 64-row groups (what one wave
// of gemm_kernel multiplies) hold 32 rows of m followed by the same 32 rows of m2, so that a lane of that wave ends up
// with both products of its (row, token) and can apply SwiGLU to them.  rows must be a multiple of 128 then.
__host__ __device__ constexpr uint32_t gemm_pair_row(uint32_t copy_row) { return copy_row / 256 * 128 + (copy_row % 256) / 64 * 32 + copy_row % 32; }
__host__ __device__ constexpr uint32_t gemm_pair_which(uint32_t copy_row) { return (copy_row % 64) / 32; }
template <int QT, bool PAIR>
__global__ __launch_bounds__(256) void expand_codes_kernel(uint16_t *__restrict__ dst, MatView m, MatView m2)
{
    const uint32_t rows_total = PAIR ? 2 * m.rows : m.rows;
    const uint32_t Kp = gemm_k_padded(m.cols), rows_pad = gemm_rows_padded(rows_total), nbp = Kp / 32, nb = m.cols / 32;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t r = (uint32_t)(t % kGemmRows);
    const uint64_t rest = t / kGemmRows;
    const uint32_t blk = (uint32_t)(rest % nbp), rt = (uint32_t)(rest / nbp);
    const uint32_t row = rt * kGemmRows + r;
    if (row >= rows_pad) return;
    const uint32_t src_row = PAIR ? gemm_pair_row(row) : row;
    const MatView &src = (PAIR && gemm_pair_which(row)) ? m2 : m;
    const bool real = row < rows_total && src_row < m.rows && blk < nb;
    _Float16 v[32];
    float d = 0.f;
    if (real) {
        const uint64_t sb = (uint64_t)src_row * nb + blk;
        d = mat_scale(src, sb);
        if constexpr (QT == 4) {
            const uint4 c = src.codes[sb];        // byte b: element b in the low nibble, element b + 16 in the high one
            const uint32_t q[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int b = 0; b < 16; b++) {
                const uint32_t byte = (q[b >> 2] >> (8 * (b & 3))) & 0xffu;
                v[b] = (_Float16)((int)(byte & 15u) - 8);
                v[b + 16] = (_Float16)((int)(byte >> 4) - 8);
            }
        } else {
            const uint4 c0 = src.codes[sb * 2], c1 = src.codes[sb * 2 + 1];
            const uint32_t q[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
#pragma unroll
            for (int b = 0; b < 32; b++) v[b] = (_Float16)(int)(int8_t)((q[b >> 2] >> (8 * (b & 3))) & 0xffu);
        }
    } else {
#pragma unroll
        for (int b = 0; b < 32; b++) v[b] = (_Float16)0.f;
    }
    const uint64_t nchunk = Kp / 8;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        union { _Float16 h[8]; uint4 u; } pk;
#pragma unroll
        for (int e = 0; e < 8; e++) pk.h[e] = v[8 * c + e];
        *reinterpret_cast<uint4 *>(dst + (((uint64_t)rt * nchunk + (uint64_t)blk * 4 + c) * kGemmRows + r) * 8) = pk.u;
    }
    float *sc = reinterpret_cast<float *>(dst + gemm_copy_code_halfs(rows_total, m.cols));
    sc[((uint64_t)rt * nbp + blk) * kGemmRows + r] = d;
}

// The steps between two GEMMs of a prompt batch as one pass over a token row: x += the K slices of the product
// before (same order as gemm_reduce_kernel: slices first, then x), xn = normalize(x) * w (normalize_kernel's
// arithmetic), and xn split in the two fp16 halves the next GEMM reads (tile order, padded to Kp with zeros).
// One 256-thread workgroup per row of the padded batch (rows as in gemm_producer_row, halves scaled as in gemm_row_scale);
// rows n.. are written as zeros.  dim <= 8192, a multiple of 8.
struct PrefillNormArgs {
    float *x;                              // [n][dim] residual stream, updated when nparts > 0
    const float *parts[kGemmMaxMats];      // [n][dim] each
    uint32_t nparts;
    const float *w;                        // norm weights
    float *xn;                             // [n][dim] or null: the normalised row as fp32 (for a GEMV-type consumer)
    uint16_t *xh, *xl;                     // tile order, n_pad x Kp
    float *xscale;                         // [n_pad]: 2^-S of the row
    uint32_t dim, n, Kp;
};
__global__ __launch_bounds__(256) void prefill_norm_kernel(PrefillNormArgs a)
{
    __shared__ float lds[4];
    constexpr int PER = 4;                 // chunks of 8 per thread
    const uint32_t row = gemm_producer_row(blockIdx.x);
    const uint32_t dim = a.dim, n8 = dim / 8;
    const bool live = row < a.n;
    const size_t ro = (size_t)(live ? row : 0) * dim;
    float v[PER][8], wv[PER][8];
    // every load of the row first (x, up to four slices, the weights: nothing depends on anything), then the sums and the
    // stores: a store between them would hold back the loads behind it, which may alias it for all the compiler knows
    float4 x4[PER][2], p4[kGemmMaxMats][PER][2];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = threadIdx.x + j * 256;
        const uint32_t ic = (live && i < n8) ? i : 0;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            const float4 w4 = reinterpret_cast<const float4 *>(a.w)[(i < n8 ? i : 0) * 2 + hf];
            wv[j][4 * hf] = w4.x; wv[j][4 * hf + 1] = w4.y; wv[j][4 * hf + 2] = w4.z; wv[j][4 * hf + 3] = w4.w;
            x4[j][hf] = reinterpret_cast<const float4 *>(a.x + ro)[ic * 2 + hf];
#pragma unroll
            for (int q = 0; q < kGemmMaxMats; q++)
                if (q < (int)a.nparts) p4[q][j][hf] = reinterpret_cast<const float4 *>(a.parts[q] + ro)[ic * 2 + hf];
        }
    }
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = threadIdx.x + j * 256;
        const bool ok = live && i < n8;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            float4 x = x4[j][hf];
            if (a.nparts) {
                float4 s4 = p4[0][j][hf];
#pragma unroll
                for (int q = 1; q < kGemmMaxMats; q++)
                    if (q < (int)a.nparts) { s4.x += p4[q][j][hf].x; s4.y += p4[q][j][hf].y; s4.z += p4[q][j][hf].z; s4.w += p4[q][j][hf].w; }
                x.x = s4.x + x.x; x.y = s4.y + x.y; x.z = s4.z + x.z; x.w = s4.w + x.w;
                if (ok) reinterpret_cast<float4 *>(a.x + ro)[i * 2 + hf] = x;
            }
            if (!ok) x = make_float4(0.f, 0.f, 0.f, 0.f);
            v[j][4 * hf] = x.x; v[j][4 * hf + 1] = x.y; v[j][4 * hf + 2] = x.z; v[j][4 * hf + 3] = x.w;
        }
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) s += ((v[j][0] + v[j][1]) + (v[j][2] + v[j][3])) + ((v[j][4] + v[j][5]) + (v[j][6] + v[j][7]));
    const float mean = block_sum_256(s, lds) / (float)dim;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        if (threadIdx.x + j * 256 < n8) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float c = v[j][e] - mean;
                q = fmaf(c, c, q);
            }
        }
    }
    const float inv = rsqrtf(block_sum_256(q, lds) / (float)dim);
    const uint32_t chunks = a.Kp / 8;
    float big = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const bool in = live && threadIdx.x + j * 256 < n8;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            v[j][e] = in ? (v[j][e] * wv[j][e]) * inv : 0.f;   // padding rows and columns: zero
            big = fmaxf(big, fabsf(v[j][e]));
        }
    }
    big = block_max_256(big, lds);
    float down;
    const float up = gemm_row_scale(big, &down);
    if (threadIdx.x == 0) a.xscale[row] = down;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = threadIdx.x + j * 256;
        if (i >= chunks) continue;
        if (live && i < n8 && a.xn) {
            reinterpret_cast<float4 *>(a.xn + ro)[i * 2] = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
            reinterpret_cast<float4 *>(a.xn + ro)[i * 2 + 1] = make_float4(v[j][4], v[j][5], v[j][6], v[j][7]);
        }
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] = v[j][e] * up;
        uint4 h, l;
        gemm_split8(h, l, f);
        const size_t o = gemm_x_offset(row, i * 8, a.Kp);
        *reinterpret_cast<uint4 *>(a.xh + o) = h;
        *reinterpret_cast<uint4 *>(a.xl + o) = l;
    }
}

// One workgroup: 128 tokens x 256 weight rows over a range of K.  The grid enumerates (matrix or K slice, row tile, token
// tile) so that the token tiles of one row tile run on one XCD (workgroups are dealt to the 8 XCDs in turn) and find its
// weights in that XCD's L2, and so that the XCDs get equal numbers of workgroups.
//
// Pipeline.  Stage s (K step s: 16 KB of weights, 2 x 8 KB of activation halves, 1 KB of scales) is copied to LDS buffer
// s % 4 by five direct loads per thread, issued three to three and a half steps before its MFMAs.  A wave holds the operands of
// the step it multiplies in registers (twelve 16-byte reads); in the second half of a step it waits for the next
// stage's loads, meets the other waves at the step's only barrier, lets the loads of stage s + 4 overwrite the buffer
// of stage s (which every wave has by then read into registers), and reads the next step's operands between its MFMAs.
// The scale multiply-adds of a 32 x 32 tile follow its last MFMA five issue slots later, four after each MFMA, so that
// neither the matrix pipe nor the vector pipe waits for the other.
// MODE 0: plain products; 1: SwiGLU of a pair copy (GemmArgs::fh); 2: plain, or fp16 rows where GemmArgs::half_out says so
template <int MODE>
__device__ __forceinline__ void gemm_body(const GemmArgs &a)
{
    constexpr bool SILU = MODE == 1;
    constexpr int TN = kGemmTile, RM = kGemmRows, NST = kGemmStages;
    constexpr int LPS = 5;   // direct loads per thread per stage
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    uint8_t *const lds = gemm_lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, wm = wave >> 2;
    const uint32_t tok_tiles = (a.n + TN - 1) / TN, row_tiles = a.tile_count ? a.tile_count : (a.rows + RM - 1) / RM;
    // unit = (matrix or slice, row tile); unit u runs on XCD u % 8, its token tiles in consecutive slots of that XCD
    const uint32_t L = blockIdx.x, xcd = L & 7, slot = L >> 3;
    const uint32_t unit = (slot / tok_tiles) * 8 + xcd, tt = slot % tok_tiles;
    if (unit >= row_tiles * a.nz) return;
    const uint32_t z = unit / row_tiles, rt = unit % row_tiles + a.tile0;
    const uint32_t Kp = gemm_k_padded(a.K), nchunk = Kp / 8, nblk = Kp / 32;
    // this workgroup's K steps: step0 .. step0 + steps - 1, an even number (slices are multiples of 64, and so is Kp)
    const uint32_t step0 = a.slice_k ? z * (a.slice_k / kGemmStep) : 0;
    const uint32_t steps = a.slice_k ? min(a.slice_k / kGemmStep, nblk - step0) : nblk;
    const uint8_t *w16 = reinterpret_cast<const uint8_t *>(a.w16[z]);
    const uint8_t *gw = w16 + ((size_t)rt * nchunk * RM + tid) * 16;
    const uint8_t *gs = w16 + gemm_copy_code_halfs(a.rows, a.K) * 2 + ((size_t)rt * nblk * RM + (wave & 3) * 64 + lane) * 4;
    const uint8_t *gh = reinterpret_cast<const uint8_t *>(a.xh) + ((size_t)tt * nchunk * TN + tid) * 16;
    const uint8_t *gl = reinterpret_cast<const uint8_t *>(a.xl) + ((size_t)tt * nchunk * TN + tid) * 16;

    // load p (0..4) of this thread's five for stage s; past the end a harmless repeat of the last stage into a free buffer,
    // which keeps the number of loads in flight the same in every step
    auto issue_one = [&](uint32_t s, int p) {
        const size_t sc = step0 + (s < steps ? s : steps - 1);
        uint8_t *buf = lds + (s % NST) * kGemmStageBytes;
        const uint8_t *pw = gw + sc * kGemmWBytes;
        if (p == 0) __builtin_amdgcn_global_load_lds((lv_glb_void *)pw, (lv_lds_void *)(buf + wave * 1024), 16, 0, 0);
        if (p == 1) __builtin_amdgcn_global_load_lds((lv_glb_void *)(pw + 8192), (lv_lds_void *)(buf + 8192 + wave * 1024), 16, 0, 0);
        if (p == 2) __builtin_amdgcn_global_load_lds((lv_glb_void *)(gh + sc * kGemmXBytes), (lv_lds_void *)(buf + kGemmWBytes + wave * 1024), 16, 0, 0);
        if (p == 3) __builtin_amdgcn_global_load_lds((lv_glb_void *)(gl + sc * kGemmXBytes), (lv_lds_void *)(buf + kGemmWBytes + kGemmXBytes + wave * 1024), 16, 0, 0);
        // scales: 1 KB, four waves' worth of 4-byte loads; waves 4..7 repeat them (same bytes to the same place)
        if (p == 4) __builtin_amdgcn_global_load_lds((lv_glb_void *)(gs + sc * kGemmScBytes), (lv_lds_void *)(buf + kGemmWBytes + 2 * kGemmXBytes + (wave & 3) * 256), 4, 0, 0);
    };

    // Accumulators: 4 x 4 tiles of 16 tokens x 16 rows (v_mfma_f32_16x16x32_f16: one instruction takes a whole quant block of
    // K = 32).  Lane l of a tile holds weight row l % 16 and, in register r, token 4 * (l / 16) + r.
    const int l15 = lane & 15, l4 = lane >> 4;
    lv_f4v acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = lv_f4v{0.f, 0.f, 0.f, 0.f};
    const lv_f4v zero = {0.f, 0.f, 0.f, 0.f};

    struct Frag { lv_h8 xh[4], xl[4], wc[4]; float d[4]; };
    // one sixth of the operand reads of a stage (two 16-byte reads: lane l takes row l % 16 of a 16-row tile, k chunk l / 16),
    // the scales with the last
    auto read_part = [&](Frag &f, const uint8_t *buf, int part) {
        const uint8_t *sW = buf, *sH = buf + kGemmWBytes, *sL = buf + kGemmWBytes + kGemmXBytes;
        const int half = part & 1, what = part >> 1;      // what: 0 weights, 1 low halves, 2 high halves
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int t = 2 * half + u;
            if (what == 0) f.wc[t] = *reinterpret_cast<const lv_h8 *>(sW + (l4 * RM + wn * 64 + t * 16 + l15) * 16);
            if (what == 1) f.xl[t] = *reinterpret_cast<const lv_h8 *>(sL + (l4 * TN + wm * 64 + t * 16 + l15) * 16);
            if (what == 2) f.xh[t] = *reinterpret_cast<const lv_h8 *>(sH + (l4 * TN + wm * 64 + t * 16 + l15) * 16);
        }
        if (part == 5) {
            const float *sD = reinterpret_cast<const float *>(buf + kGemmWBytes + 2 * kGemmXBytes);
#pragma unroll
            for (int j = 0; j < 4; j++) f.d[j] = sD[wn * 64 + j * 16 + l15];
        }
    };
    // A step = 32 MFMA slots: tile t (token tile t / 4, row tile t % 4) takes two, low halves first (from zero), then high
    // halves on top; tiles go in pairs (L0 L1 H0 H1 L2 L3 ...), so that no MFMA waits for the one before it.  The scale
    // multiply-adds, two per slot, follow in tile order four slots behind: tile t's four in slots 4 + 2t and 5 + 2t, at least two
    // slots after its second MFMA was issued.  Those of tiles 14 and 15 fall into the first four slots of the next step (cv, cd).
    float cv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, cd[2] = {0.f, 0.f};
    auto step = [&](uint32_t s, const Frag &cur, Frag &nxt) {
        lv_f4v T[16];
#pragma unroll
        for (int g = 0; g < 32; g++) {
            if (g == 16) {
                // stage s + 1 has landed for everyone, and everyone holds stage s in registers: from here on its buffer may
                // take stage s + 4
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 2) * LPS) : "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            const int t = g >> 1, ti = t >> 2, tj = t & 3;
            if ((g & 1) == 0) T[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cur.xl[ti], cur.wc[tj], zero, 0, 0, 0);
            else T[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cur.xh[ti], cur.wc[tj], T[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 2; e++) {
                if (g < 4) {
                    const int idx = 2 * g + e;      // tiles 14 and 15 of the step before: token tile 3, row tiles 2 and 3
                    acc[3][2 + (idx >> 2)][idx & 3] = fmaf(cv[idx], cd[idx >> 2], acc[3][2 + (idx >> 2)][idx & 3]);
                } else {
                    const int k = 2 * (g - 4) + e, q = k >> 2, r = k & 3;
                    acc[q >> 2][q & 3][r] = fmaf(T[q][r], cur.d[q & 3], acc[q >> 2][q & 3][r]);
                }
            }
            if (g >= 16 && g < 22) read_part(nxt, lds + ((s + 1) % NST) * kGemmStageBytes, g - 16);
            // the five loads of stage s + 4, one at a time between the MFMAs of this step's second half and the next step's
            // first: issued together right behind the barrier, the forty of a workgroup back up and hold the waves that
            // issue them, MFMAs included
            if (g == 18) issue_one(s + NST, 0);
            if (g == 24) issue_one(s + NST, 1);
            if (g == 30) issue_one(s + NST, 2);
            if (g == 4) issue_one(s + NST - 1, 3);
            if (g == 10) issue_one(s + NST - 1, 4);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) { cv[r] = T[14][r]; cv[4 + r] = T[15][r]; }
        cd[0] = cur.d[2]; cd[1] = cur.d[3];
    };
    Frag FA, FB;
#pragma unroll
    for (int s = 0; s < NST; s++)
#pragma unroll
        for (int p = 0; p < (s == NST - 1 ? 3 : LPS); p++) issue_one(s, p);      // the last two of stage 3 follow in step 0
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 1) * LPS - 2) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int p = 0; p < 6; p++) read_part(FA, lds, p);
    for (uint32_t s = 0; s < steps; s += 2) {
        step(s, FA, FB);
        step(s + 1, FB, FA);
    }
#pragma unroll
    for (int idx = 0; idx < 8; idx++) acc[3][2 + (idx >> 2)][idx & 3] = fmaf(cv[idx], cd[idx >> 2], acc[3][2 + (idx >> 2)][idx & 3]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // the repeats past the end have landed before the workgroup gives up its LDS

    // acc[ti][tj][r]: token tt * 128 + wm * 64 + ti * 16 + 4 * l4 + r, weight row rt * 256 + wn * 64 + tj * 16 + l15.
    // The per-token scales of this lane's 16 tokens, fetched before the first store (the stores may alias them for all the
    // compiler knows, and a load behind every store costs the launch 6 us)
    float4 ts[4];
#pragma unroll
    for (int ti = 0; ti < 4; ti++) {
        ts[ti] = make_float4(1.f, 1.f, 1.f, 1.f);
        if (a.xscale) ts[ti] = *reinterpret_cast<const float4 *>(a.xscale + tt * TN + wm * 64 + ti * 16 + 4 * l4);   // n_pad entries: in range
    }
    auto tscale = [&](int ti, int r) { return r == 0 ? ts[ti].x : r == 1 ? ts[ti].y : r == 2 ? ts[ti].z : ts[ti].w; };
    if constexpr (SILU) {
        // row tiles 0, 1 = gate rows, 2, 3 = the same up rows: this lane's ff values of rows rt * 128 + wn * 32 + tj * 16 + l15
        // (tj = 0, 1) and its 16 tokens.  They pass through LDS (per wave: [64 tokens][32 rows] halfs, high and low apart) to
        // come out as 16-byte chunks of 8 consecutive rows of one token, consecutive lanes taking consecutive tokens: what a
        // chunk row of the down projection's activation tile is.  Padding tokens give 0 * 0 / 2 = 0, as their rows of the
        // tile must be.
        constexpr int TS = 80;                      // bytes per token in the exchange: 64 + 16, so that 8 lanes' 16-byte reads miss each other's banks
        __syncthreads();                            // every wave holds its last operands in registers: the stages are free
        uint8_t *xb = lds + wave * (2 * 64 * TS);
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int tj = 0; tj < 2; tj++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int tok = ti * 16 + 4 * l4 + r;
                    const float sc = tscale(ti, r);
                    const float g = acc[ti][tj][r] * sc, u = acc[ti][tj + 2][r] * sc;
                    const float f = g * u / (__expf(-u) + 1.f);
                    const uint16_t h = float_to_half_bits(f), l = float_to_half_bits(f - half_bits_to_float(h));
                    *reinterpret_cast<uint16_t *>(xb + tok * TS + (tj * 16 + l15) * 2) = h;
                    *reinterpret_cast<uint16_t *>(xb + 64 * TS + tok * TS + (tj * 16 + l15) * 2) = l;
                }
        __syncthreads();
        const uint32_t n = tt * TN + wm * 64 + lane;                  // below n_pad: the token tiles cover the padded batch
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint4 hv = *reinterpret_cast<const uint4 *>(xb + lane * TS + c * 16), lv = *reinterpret_cast<const uint4 *>(xb + 64 * TS + lane * TS + c * 16);
            const size_t o = gemm_x_offset(n, rt * 128 + wn * 32 + c * 8, a.fKp);
            *reinterpret_cast<uint4 *>(a.fh + o) = hv;
            *reinterpret_cast<uint4 *>(a.fl + o) = lv;
        }
        return;
    }
    if constexpr (MODE == 2) {
        if (a.half_out[z]) {
            // the wave's 64 tokens x 64 rows pass through LDS as halfs ([token][row], 128 + 16 bytes a token) and leave as 16-byte
            // chunks of 8 consecutive rows, eight lanes on the 128 bytes of a token
            constexpr int TS = 144;
            __syncthreads();                            // every wave holds its last operands in registers: the stages are free
            uint8_t *xb = lds + wave * (64 * TS);
#pragma unroll
            for (int ti = 0; ti < 4; ti++)
#pragma unroll
                for (int tj = 0; tj < 4; tj++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int tok = ti * 16 + 4 * l4 + r;
                        *reinterpret_cast<uint16_t *>(xb + tok * TS + (tj * 16 + l15) * 2) = float_to_half_bits(acc[ti][tj][r] * tscale(ti, r));
                    }
            __syncthreads();
            const uint32_t row0 = (a.row_ptr ? *a.row_ptr : 0u) + a.row_add;
            uint16_t *const dst = a.half_out[z];
#pragma unroll
            for (int it = 0; it < 8; it++) {
                const int tok = it * 8 + (lane >> 3), c = lane & 7;
                const uint32_t n = tt * TN + wm * 64 + tok, m = rt * RM + wn * 64 + c * 8;
                const uint4 v = *reinterpret_cast<const uint4 *>(xb + tok * TS + c * 16);
                if (n < a.n && m < a.rows && row0 + n < a.row_limit) *reinterpret_cast<uint4 *>(dst + (size_t)(row0 + n) * a.ldo + m) = v;
            }
            return;
        }
    }
    float *const out = a.outs[z];
#pragma unroll
    for (int ti = 0; ti < 4; ti++)
#pragma unroll
        for (int tj = 0; tj < 4; tj++) {
            const uint32_t m = rt * RM + wn * 64 + tj * 16 + l15;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t n = tt * TN + wm * 64 + ti * 16 + 4 * l4 + r;
                if (n < a.n && m < a.rows) {
                    float *dst = out + (size_t)n * a.ldo + (m - a.tile0 * RM);
                    const float v = acc[ti][tj][r] * tscale(ti, r);
                    *dst = a.accumulate ? *dst + v : v;
                }
            }
        }
}

template <bool SILU>
__global__ __launch_bounds__(512) void gemm_kernel(GemmArgs a)
{
    gemm_body<SILU ? 1 : 0>(a);
}

// q, k and v of a prompt batch in one launch: q as fp32 rows, k and v as fp16 rows of their caches (GemmArgs::half_out)
__global__ __launch_bounds__(512) void gemm_rows16_kernel(GemmArgs a)
{
    gemm_body<2>(a);
}

}  // namespace lv
