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
// Tiling: workgroup = 8 (or 4) waves, output tile 128 tokens x 128 (or 64) weight rows, K step 64 (two quant blocks).
// Two threads unpack one (row, block) pair per step; every wave owns a 32-token x 64-row sub-tile of
// v_mfma_f32_32x32x16_f16 tiles.  The global loads of step s+2 are issued before the MFMAs of step s.
#pragma once

#include "lv_kernels.h"

namespace lv {

typedef _Float16 lv_h8 __attribute__((ext_vector_type(8)));
typedef float lv_f16v __attribute__((ext_vector_type(16)));

constexpr int kGemmTile = 128;  // tokens per workgroup (batches are padded to multiples of it)
constexpr int kGemmK = 64;      // K per step
constexpr int kGemmLd = kGemmK + 8;  // LDS row stride in halfs (the pad spreads 16-byte reads over the banks)

// x[n][K] fp32 -> xh, xl [n_pad][K] fp16 (rows n..n_pad-1 zero).  Inside every 32-element block the halves are stored
// in the order the GEMM for weight type QT keeps its weight halves in (gemm_k_position).
template <int QT>
__global__ void split_half_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, const float *__restrict__ x, uint32_t n, uint32_t K)
{
    const uint32_t row = blockIdx.y;
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= K) return;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < n) v = *reinterpret_cast<const float4 *>(x + (size_t)row * K + i);
    const float f[4] = {v.x, v.y, v.z, v.w};
    const uint32_t blk0 = i & ~31u, e0 = i & 31u;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint16_t h = float_to_half_bits(f[j]);
        const uint16_t l = float_to_half_bits(f[j] - half_bits_to_float(h));
        int pos = (int)e0 + j;
        if constexpr (QT == 4) {
            const int hi = pos >= 16 ? 1 : 0, ee = pos & 15, ii = ee >> 2, b = ee & 3;
            pos = 8 * ii + 2 * ((b & 1) * 2 + hi) + (b >> 1);
        }
        xh[(size_t)row * K + blk0 + pos] = h;
        xl[(size_t)row * K + blk0 + pos] = l;
    }
}

constexpr int kGemmMaxMats = 3;
struct GemmArgs {
    // up to three matrices of one shape and type applied to the same activations in one launch (blockIdx.z picks the
    // matrix): q, k and v of a layer together fill the CUs that each alone leaves idle
    float *outs[kGemmMaxMats];  // [n][ldo] each
    const uint16_t *xh, *xl;  // [n_pad][K] fp16 halves of the activations, n_pad a multiple of 128
    MatView ws[kGemmMaxMats];   // rows x K each
    uint32_t n;             // tokens
    uint32_t ldo;           // floats between output rows
    int accumulate;         // out += instead of out =
    // 0: blockIdx.z picks the matrix.  Otherwise the launch splits K: ws[] all name one matrix, slice z multiplies the
    // K steps z*slice_steps .. (z+1)*slice_steps-1 into outs[z], and gemm_reduce_kernel adds the slices up (a matrix
    // with few rows and a long K, like the down projection, fills the CUs that way)
    uint32_t slice_steps;
};

// out[n][ldo] (+)= p[0] + p[1] (+ p[2]), the K slices of one product, each [n][rows]; always summed in this order
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

typedef _Float16 lv_h2 __attribute__((ext_vector_type(2)));

// Position inside a 32-element block at which the weight halves of element e are stored in LDS, and therefore at
// which the activation halves must be stored too (split_half_kernel).  q8_0: natural order.  q4_0: the order in
// which whole dwords of codes unpack into pairs of fp16 — dword i, shift 4j holds elements (4i, 4i+2), (16+4i, 18+4i),
// (4i+1, 4i+3), (17+4i, 19+4i) for j = 0..3 (byte b of a block carries element b in its low and b+16 in its high nibble).
template <int QT>
__host__ __device__ constexpr int gemm_k_position(int e)
{
    if (QT != 4) return e;
    const int hi = e >= 16 ? 1 : 0, ee = e & 15, i = ee >> 2, b = ee & 3;
    const int j = (b & 1) * 2 + hi;
    return 8 * i + 2 * j + (b >> 1);
}

// 16 codes of half a block (q8_0: 16 bytes; q4_0: 8 bytes, the two dwords whose nibbles unpack to positions
// 16*half .. 16*half+15 of gemm_k_position order) -> 16 halfs at w, as the integers they are (q4_0: q - 8, q8_0: q):
// 1024 + u has the fp16 bit pattern 0x6400 | u, and subtracting 1024 + offset is exact.  A block outside the matrix
// is given the scale 0 by the caller, which removes it from the sum whatever codes were unpacked for it.
template <int QT, typename CW>
__device__ __forceinline__ void gemm_codes_half(uint16_t *w, const CW &c)
{
    uint32_t ph[8];
    auto emit = [&](int slot, uint32_t packed_codes, _Float16 bias) {
        // packed_codes: two halfs 0x6400 | u
        union { uint32_t u; lv_h2 h; } cc, v;
        cc.u = packed_codes;
        const lv_h2 bb = {bias, bias};
        v.h = cc.h - bb;                             // exact: small integers
        ph[slot] = v.u;
    };
    if constexpr (QT == 4) {
        const uint32_t q[2] = {c.x, c.y};
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) emit(4 * i + j, ((q[i] >> (4 * j)) & 0x000f000fu) | 0x64006400u, (_Float16)1032.f);
    } else {
        const uint32_t q[4] = {c.x, c.y, c.z, c.w};      // CW = uint4
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t u = q[i] ^ 0x80808080u;   // int8 -> biased unsigned
            // one byte permute per pair: bytes (u.b0, 0x64, u.b1, 0x64) and (u.b2, 0x64, u.b3, 0x64)
            emit(2 * i, __builtin_amdgcn_perm(u, 0x64646464u, 0x00050004u), (_Float16)1152.f);
            emit(2 * i + 1, __builtin_amdgcn_perm(u, 0x64646464u, 0x00070006u), (_Float16)1152.f);
        }
    }
#pragma unroll
    for (int g = 0; g < 2; g++) *reinterpret_cast<uint4 *>(w + 8 * g) = make_uint4(ph[4 * g], ph[4 * g + 1], ph[4 * g + 2], ph[4 * g + 3]);
}

// ff[n][F] = a * b / (exp(-b) + 1) (matmul_silu_ff.comp:96 with a = W3 x, b = W1 x), written as the two fp16 halves
// the down projection's GEMM reads (split_half_kernel's layout for weight type QT; rows n.. zero)
template <int QT>
__global__ void silu_split_kernel(uint16_t *__restrict__ xh, uint16_t *__restrict__ xl, const float *__restrict__ a, const float *__restrict__ b,
                                  uint32_t n, uint32_t K)
{
    const uint32_t row = blockIdx.y;
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= K) return;
    float f[4] = {0.f, 0.f, 0.f, 0.f};
    if (row < n) {
        const float4 r1 = *reinterpret_cast<const float4 *>(a + (size_t)row * K + i), r2 = *reinterpret_cast<const float4 *>(b + (size_t)row * K + i);
        f[0] = r1.x * r2.x / (__expf(-r2.x) + 1.f);
        f[1] = r1.y * r2.y / (__expf(-r2.y) + 1.f);
        f[2] = r1.z * r2.z / (__expf(-r2.z) + 1.f);
        f[3] = r1.w * r2.w / (__expf(-r2.w) + 1.f);
    }
    const uint32_t blk0 = i & ~31u, e0 = i & 31u;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint16_t h = float_to_half_bits(f[j]);
        const uint16_t l = float_to_half_bits(f[j] - half_bits_to_float(h));
        const int pos = gemm_k_position<QT>((int)e0 + j);
        xh[(size_t)row * K + blk0 + pos] = h;
        xl[(size_t)row * K + blk0 + pos] = l;
    }
}

// The steps between two GEMMs of a prompt batch as one pass over a token row: x += the K slices of the product
// before (same order as gemm_reduce_kernel: slices first, then x), xn = normalize(x) * w (normalize_kernel's
// arithmetic), and xn split in the two fp16 halves the next GEMM reads (split_half_kernel's layout for weight type QT).
// One 256-thread workgroup per row of the padded batch; rows n.. are written as zeros.  dim <= 8192, a multiple of 4.
struct PrefillNormArgs {
    float *x;                              // [n][dim] residual stream, updated when nparts > 0
    const float *parts[kGemmMaxMats];      // [n][dim] each
    uint32_t nparts;
    const float *w;                        // norm weights
    float *xn;                             // [n][dim] or null: the normalised row as fp32 (for a GEMV-type consumer)
    uint16_t *xh, *xl;                     // [n_pad][dim]
    uint32_t dim, n;
};
template <int QT>
__global__ __launch_bounds__(256) void prefill_norm_kernel(PrefillNormArgs a)
{
    __shared__ float lds[4];
    constexpr int PER = 8;
    const uint32_t row = blockIdx.x, dim = a.dim, n4 = dim / 4;
    const bool live = row < a.n;
    const size_t ro = (size_t)(live ? row : 0) * dim;
    float4 v[PER], wv[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = threadIdx.x + j * 256;
        const bool ok = live && i < n4;
        const uint32_t ic = ok ? i : 0;
        wv[j] = reinterpret_cast<const float4 *>(a.w)[i < n4 ? i : 0];
        float4 x4 = reinterpret_cast<const float4 *>(a.x + ro)[ic];
        if (a.nparts) {
            float4 s4 = reinterpret_cast<const float4 *>(a.parts[0] + ro)[ic];
            for (uint32_t q = 1; q < a.nparts; q++) {
                const float4 p4 = reinterpret_cast<const float4 *>(a.parts[q] + ro)[ic];
                s4.x += p4.x; s4.y += p4.y; s4.z += p4.z; s4.w += p4.w;
            }
            x4.x = s4.x + x4.x; x4.y = s4.y + x4.y; x4.z = s4.z + x4.z; x4.w = s4.w + x4.w;
            if (ok) reinterpret_cast<float4 *>(a.x + ro)[ic] = x4;
        }
        v[j] = ok ? x4 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    const float mean = block_sum_256(s, lds) / (float)dim;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        if (threadIdx.x + j * 256 < n4) {
            const float c0 = v[j].x - mean, c1 = v[j].y - mean, c2 = v[j].z - mean, c3 = v[j].w - mean;
            q = fmaf(c0, c0, q); q = fmaf(c1, c1, q); q = fmaf(c2, c2, q); q = fmaf(c3, c3, q);
        }
    }
    const float inv = rsqrtf(block_sum_256(q, lds) / (float)dim);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = threadIdx.x + j * 256;
        if (i >= n4) continue;
        float f[4] = {(v[j].x * wv[j].x) * inv, (v[j].y * wv[j].y) * inv, (v[j].z * wv[j].z) * inv, (v[j].w * wv[j].w) * inv};
        if (!live) f[0] = f[1] = f[2] = f[3] = 0.f;        // a padding row (its inv is not finite)
        if (live && a.xn) reinterpret_cast<float4 *>(a.xn + ro)[i] = make_float4(f[0], f[1], f[2], f[3]);
        const uint32_t e = i * 4, blk0 = e & ~31u, e0 = e & 31u;
        uint16_t *hr = a.xh + (size_t)row * dim + blk0, *lr = a.xl + (size_t)row * dim + blk0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint16_t h = float_to_half_bits(f[k]);
            const uint16_t l = float_to_half_bits(f[k] - half_bits_to_float(h));
            const int pos = gemm_k_position<QT>((int)e0 + k);
            hr[pos] = h;
            lr[pos] = l;
        }
    }
}

// RM = weight rows per workgroup (128 or 64); tokens per workgroup: 128.  The four waves split the tile 2 x 2
// (RM = 128: 64 tokens x 64 rows each) or 4 x 1 (RM = 64: 32 tokens x 64 rows each).  The narrow form doubles the
// number of workgroups for matrices that would otherwise not fill 256 CUs.
template <int QT, int RM, int NWV = 4, bool SF32 = false /* fp32 scale plane (file version 1) */, bool DB = false /* two LDS buffers */>
__global__ __launch_bounds__(NWV * 64) void gemm_kernel(GemmArgs a)
{
    constexpr int TN = kGemmTile;                 // tokens per workgroup
    constexpr int WN = RM / 64;                   // waves along the rows
    constexpr int WM = NWV / WN;                  // waves along the tokens
    constexpr int NT = NWV * 64;                  // threads
    constexpr int XP = TN * 8 / NT;               // 16-byte pieces of an activation half-tile per thread
    constexpr int MT = TN / WM / 32;              // 32-token tiles per wave
    constexpr int NBUF = DB ? 2 : 1;
    __shared__ __attribute__((aligned(16))) uint16_t sXh_[NBUF][TN * kGemmLd], sXl_[NBUF][TN * kGemmLd], sW_[NBUF][RM * kGemmLd];
    __shared__ float sD_[NBUF][2][RM];            // scale of (block of the step, row)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const uint32_t tok0 = blockIdx.y * TN, row0 = blockIdx.x * RM;
    const MatView w = a.ws[blockIdx.z];
    float *const out = a.outs[blockIdx.z];
    const uint32_t K = w.cols, nb = K / 32, all_steps = (K + kGemmK - 1) / kGemmK;
    // this workgroup's K steps: step0 .. step0 + steps - 1 (the host gives every slice at least one)
    const uint32_t step0 = a.slice_steps ? blockIdx.z * a.slice_steps : 0;
    const uint32_t steps = a.slice_steps ? min(a.slice_steps, all_steps - step0) : all_steps;

    // this thread's share of the weights of a step: half h_w of block (2*step + b_w) of row r_w.  Every thread has one,
    // and every load below is issued by every thread at every step (addresses are clamped, results discarded where
    // there is nothing to load): the compiler can then count the loads in flight exactly and wait for the oldest set
    // only, which a load under a condition would force it to give up.
    static_assert(RM * 4 % NT == 0, "two threads per (row, block)");
    constexpr int WP = RM * 4 / NT;               // (row, block, half) pieces per thread: rows r_w + (NT/4)*i
    const int r_w = tid >> 2, b_w = (tid >> 1) & 1, h_w = tid & 1;
    // this thread's 16-byte pieces of the activation tile of a step: token rows tid/8 + XR*i, halfs (tid%8)*8..+7
    const int xr = tid >> 3, xc = (tid & 7) * 8;
    constexpr int XR = NT / 8;                    // token rows covered per piece index
    const uint32_t steps2 = (steps + 1) & ~1u;    // the loop takes two steps at a time; a step past the end multiplies zeros

    // two register sets: the loads of step s + 2 are in flight while step s is multiplied (one step of MFMAs is
    // shorter than a trip to memory)
    using CodeWords = typename std::conditional<QT == 8, uint4, uint2>::type;     // 16 codes
    // register sets of the two-buffer form: three (loads two and three steps ahead) where they fit; the 256-row q4_0
    // form would spill with three and runs with two (loads two steps ahead, issued after the unpacking instead of
    // before it), which costs q8_0 8 % but is 12 % faster than the 128-row form for q4_0
    constexpr int kSets = (QT == 4 && RM == 256) ? 2 : 3;
    struct Staged {
        CodeWords c[WP];
        uint32_t dbits[WP]; // raw scale word
        bool wvalid[WP];
        uint4 gh[XP], gl[XP];
    } pre[DB ? kSets : 2];
    auto fetch = [&](Staged &p, uint32_t step) {
        const bool real = step < steps;
        const uint32_t sc = step0 + (real ? step : steps - 1);
        const uint32_t blk = 2 * sc + b_w;
#pragma unroll
        for (int i = 0; i < WP; i++) {
            const uint32_t wrow = row0 + r_w + (NT / 4) * i;
            p.wvalid[i] = real && wrow < w.rows && blk < nb;
            const size_t sb = (size_t)(p.wvalid[i] ? wrow : 0) * nb + (p.wvalid[i] ? blk : 0);
            if constexpr (QT == 8) {
                p.c[i] = w.codes[sb * 2 + h_w];
            } else {
                p.c[i] = reinterpret_cast<const uint2 *>(w.codes)[sb * 2 + h_w];
            }
            if constexpr (SF32) p.dbits[i] = __float_as_uint(w.scales_f32[sb]);
            else p.dbits[i] = w.scales[sb];
        }
        const uint32_t k = sc * kGemmK + xc;
        const bool kok = real && k < K;
#pragma unroll
        for (int i = 0; i < XP; i++) {
            const size_t off = (size_t)(tok0 + xr + XR * i) * K + (kok ? k : 0);
            p.gh[i] = *reinterpret_cast<const uint4 *>(a.xh + off);
            p.gl[i] = *reinterpret_cast<const uint4 *>(a.xl + off);
            if (!kok) p.gh[i] = p.gl[i] = make_uint4(0, 0, 0, 0);
        }
    };

    lv_f16v acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    fetch(pre[0], 0);
    // registers -> LDS buffer `buf`
    auto stage = [&](const Staged &P, int buf) {
        uint16_t *sXh = sXh_[buf], *sXl = sXl_[buf], *sW = sW_[buf];
#pragma unroll
        for (int i = 0; i < WP; i++) {
            const int r = r_w + (NT / 4) * i;
            gemm_codes_half<QT>(sW + r * kGemmLd + b_w * 32 + h_w * 16, P.c[i]);
            if (h_w == 0) sD_[buf][b_w][r] = !P.wvalid[i] ? 0.f : SF32 ? __uint_as_float(P.dbits[i]) : half_bits_to_float((uint16_t)P.dbits[i]);
        }
#pragma unroll
        for (int i = 0; i < XP; i++) {
            *reinterpret_cast<uint4 *>(sXh + (xr + XR * i) * kGemmLd + xc) = P.gh[i];
            *reinterpret_cast<uint4 *>(sXl + (xr + XR * i) * kGemmLd + xc) = P.gl[i];
        }
    };
    // the step held by LDS buffer `buf` into the accumulators
    auto multiply = [&](int buf) {
        const uint16_t *sXh = sXh_[buf], *sXl = sXl_[buf], *sW = sW_[buf];
#pragma unroll
        for (int b = 0; b < kGemmK / 32; b++) {          // the two quant blocks of the step
            lv_f16v blk[MT][2];
#pragma unroll
            for (int i = 0; i < MT; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) blk[i][j][r] = 0.f;
#pragma unroll
            for (int kk = 2 * b; kk < 2 * b + 2; kk++) {
                const int ko = kk * 16 + (lane >> 5) * 8;
                lv_h8 xh[MT], xl[MT], wc[2];
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const int xrow = (wm * MT + t) * 32 + (lane & 31);
                    xh[t] = *reinterpret_cast<const lv_h8 *>(sXh + xrow * kGemmLd + ko);
                    xl[t] = *reinterpret_cast<const lv_h8 *>(sXl + xrow * kGemmLd + ko);
                }
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const int wr = wn * 64 + t * 32 + (lane & 31);
                    wc[t] = *reinterpret_cast<const lv_h8 *>(sW + wr * kGemmLd + ko);
                }
                // product by product over all tiles: consecutive MFMAs do not wait for each other's accumulator
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) blk[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl[i], wc[j], blk[i][j], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) blk[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh[i], wc[j], blk[i][j], 0, 0, 0);
            }
            // times the block's scale: a lane's sixteen results of a tile belong to one weight row
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float d = sD_[buf][b][wn * 64 + j * 32 + (lane & 31)];
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(blk[i][j][r], d, acc[i][j][r]);
            }
        }
    };
    if constexpr (!DB) {
        // one buffer: unpack, barrier, multiply, barrier; two register sets, the loads of step s + 2 in flight
        fetch(pre[1], 1);
        auto one_step = [&](Staged &P, uint32_t step) {
            stage(P, 0);
            __syncthreads();
            fetch(P, step + 2);
            multiply(0);
            __syncthreads();
        };
        for (uint32_t step = 0; step < steps2; step += 2) {
            one_step(pre[0], step);
            one_step(pre[1], step + 1);
        }
    } else {
        // two buffers, one barrier per step: step s + 1 is unpacked into one buffer while step s is multiplied out of
        // the other, so a wave's unpacking sits between its MFMAs; three register sets, the loads of steps s + 2 and
        // s + 3 in flight
        if constexpr (kSets == 2) {
            fetch(pre[1], 1);
            stage(pre[0], 0);
            fetch(pre[0], 2);
            __syncthreads();
            auto it2 = [&](uint32_t s, Staged &next) {
                stage(next, (s + 1) & 1);
                fetch(next, s + 3);
                multiply(s & 1);
                __syncthreads();
            };
            for (uint32_t s = 0; s < steps; s += 2) {
                it2(s, pre[1]);
                if (s + 1 >= steps) break;
                it2(s + 1, pre[0]);
            }
        } else {
        fetch(pre[1], 1);
        fetch(pre[kSets - 1], 2);
        stage(pre[0], 0);
        __syncthreads();
        // mine: the set that held step s (in LDS since the iteration before), reloaded with step s + 3;
        // next: the set holding step s + 1
        auto iteration = [&](uint32_t s, Staged &mine, const Staged &next) {
            fetch(mine, s + 3);
            stage(next, (s + 1) & 1);
            multiply(s & 1);
            __syncthreads();
        };
        for (uint32_t s = 0; s < steps; s += 6) {
            iteration(s, pre[0], pre[1]);
            if (s + 1 >= steps) break;
            iteration(s + 1, pre[1], pre[kSets - 1]);
            if (s + 2 >= steps) break;
            iteration(s + 2, pre[kSets - 1], pre[0]);
            if (s + 3 >= steps) break;
            iteration(s + 3, pre[0], pre[1]);
            if (s + 4 >= steps) break;
            iteration(s + 4, pre[1], pre[kSets - 1]);
            if (s + 5 >= steps) break;
            iteration(s + 5, pre[kSets - 1], pre[0]);
        }
        }
    }

    // D[i][j]: i = token within the 32-tile, j = weight row; lane l holds j = l%32 and, in register r,
    // i = 8*(r/4) + 4*(l/32) + r%4
#pragma unroll
    for (int ti = 0; ti < MT; ti++)
#pragma unroll
        for (int tj = 0; tj < 2; tj++) {
            const uint32_t m = row0 + wn * 64 + tj * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t n = tok0 + (wm * MT + ti) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (n < a.n && m < w.rows) {
                    float *dst = out + (size_t)n * a.ldo + m;
                    *dst = a.accumulate ? *dst + acc[ti][tj][r] : acc[ti][tj][r];
                }
            }
        }
}

}  // namespace lv
