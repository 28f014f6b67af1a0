// lv_gemv_wide.h — the dequant-fused GEMV for matrices large enough to occupy the whole chip (one launch = one
// matrix, the shapes of matmul.glsl / matmul_silu_ff.comp at LLaMA sizes).
//
// Same streaming scheme as the phases of the persistent kernel: up to 256 workgroups of 12 wavefronts, the input
// vector staged once per workgroup in LDS, every wavefront bound to one 64-block column slab (its lanes keep
// their 32 activations in registers) and walking its share of the workgroup's rows with a register queue of
// loads kept four rows ahead.  The small-workgroup kernel in lv_kernels.h re-reads x for every 4-16 rows and has
// one row's loads in flight per wave; at 4096 x 11008 that costs more time than the weights themselves.
#pragma once

#include "lv_kernels.h"

namespace lv {

constexpr int kWideWaves = 12;
// rows requested ahead per wave.  Eight was measured too: slower at 4096 rows (a row set is then three rows long and
// most of the queue's first turn is empty), no faster at 32000.
template <int QT, int NMAT> constexpr int kWideDepth = 4;
constexpr int kWideMaxK = 64 * 32 * kWideWaves;   // widest row: every wave one slab (24576 columns)

struct WideTile {
    uint4 c, c2;
    uint32_t d;     // raw scale word (fp16 bits, or fp32 bits for a version-1 file)
};

// SF32: the matrix has an fp32 scale plane (file version 1).  A template parameter, not a test of the view: a branch
// per tile would stand between the loads of the queue, and the queue only runs ahead through straight-line code.
// NT: non-temporal loads for the q4_0 codes (the gate and up projection, whose two matrices together are the largest stream
// of a layer: 16.0 -> 15.1 us at the 7B shape; the 4096 x 4096 launches lose with them, 5.8 -> 6.5 us).
template <int QT, bool SF32, bool NT = false>
__device__ __forceinline__ void wide_load(WideTile &t, const MatView &m, uint64_t blk, bool ok)
{
    const uint64_t b = ok ? blk : 0;     // rows / lanes without a block read block 0 and are discarded
    if constexpr (QT == 4 && NT) {
        typedef uint32_t nt_u4v __attribute__((ext_vector_type(4)));
        const nt_u4v v = __builtin_nontemporal_load(reinterpret_cast<const nt_u4v *>(m.codes + b));
        t.c = make_uint4(v.x, v.y, v.z, v.w);
    } else if constexpr (QT == 4) {
        t.c = m.codes[b];
    } else {
        t.c = m.codes[2 * b];
        t.c2 = m.codes[2 * b + 1];
    }
    if constexpr (SF32) t.d = __float_as_uint(m.scales_f32[b]);
    else t.d = m.scales[b];
}

template <int QT, bool SF32>
__device__ __forceinline__ float wide_dot(const WideTile &t, const float (&x)[32], float xsum)
{
    const float d = SF32 ? __uint_as_float(t.d) : half_bits_to_float((uint16_t)t.d);
    if constexpr (QT == 4) return (q4_block_dot(t.c, x) - 8.f * xsum) * d;
    else return (q8_block_dot(t.c, t.c2, x) - 128.f * xsum) * d;
}

// Workgroup barrier that orders LDS traffic only: the weight loads in flight stay in flight.
__device__ __forceinline__ void wide_lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The input vector sits in LDS block by block (32 floats = 128 bytes) and lane l of a wave reads block 64 * slab + l: in
// plain order the 64 lanes of a 128-bit read would all fall on the same four banks.  Inside each block the eight 16-byte
// groups are therefore rotated by the block index: offset of the four floats starting at element i (a multiple of 4).
__device__ __forceinline__ uint32_t wide_xs_offset(uint32_t i)
{
    return (i & ~31u) | ((((i >> 2) + (i >> 5)) & 7u) << 2);
}

// sum over the workgroup through kWideWaves floats of LDS (one barrier; the caller alternates scratch areas)
__device__ __forceinline__ float wide_block_sum(float v, float *scratch, int w, int lane)
{
    v = wave_sum(v);
    if (lane == 0) scratch[w] = v;
    wide_lds_barrier();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kWideWaves; i++) t += scratch[i];
    return t;
}

// NMAT = 2: the SiLU form, rows of w (W3) and w1 (W1) with the same index are walked together.
template <int QT, int MODE, bool SF32>
__device__ __forceinline__ void gemv_wide_body(const GemvArgs &a, uint32_t rows_per_wg, uint32_t z /* batch row */, float *xs, float *red,
                                               float *stat /* 32 floats */)
{
    constexpr int NMAT = MODE == kGemvSilu ? 2 : 1;
    constexpr int NW = kWideWaves;
    const uint32_t N = a.w.rows, K = a.w.cols, nb = K / 32;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int NS = (int)((nb + 63) / 64), NR = NW / NS;        // slabs; row sets (waves sharing a slab split the rows)
    const int slab = w % NS, rset = w / NS;
    const bool active = rset < NR;
    const uint32_t blk_col = (uint32_t)slab * 64 + lane;
    const bool lane_ok = active && blk_col < nb;
    const uint32_t row0 = blockIdx.x * rows_per_wg;
    const uint32_t n_rows = row0 < N ? min(rows_per_wg, N - row0) : 0;
    const uint32_t per_set = (rows_per_wg + NR - 1) / NR;       // rows per row set (static upper bound)

    // the first rows' loads go out before anything else
    constexpr int DEPTH = kWideDepth<QT, NMAT>;
    WideTile q[NMAT][DEPTH];
    auto fetch = [&](int slot, uint32_t i) {       // i = index of the row inside this wave's row set
        const uint32_t r = (uint32_t)rset * per_set + i;
        const bool ok = lane_ok && i < per_set && r < n_rows;
        const uint64_t blk = (uint64_t)(row0 + r) * nb + blk_col;
        wide_load<QT, SF32, NMAT == 2>(q[0][slot], a.w, blk, ok);
        if constexpr (NMAT == 2) wide_load<QT, SF32, true>(q[1][slot], a.w1, blk, ok);
    };
#pragma unroll
    for (int i = 0; i < DEPTH; i++) fetch(i, i);

    // ---- x -> LDS -> registers; optionally normalised on the way (normalize.comp:34-64) ---------------------------
    // With norm weights, LDS gets x*w and the scalar rsqrt(mean((x - mean)^2)) multiplies the row sums at the end.
    const float *xz = a.x + (size_t)z * K;
    float inv = 1.f;
    if (a.norm_w) {
        float s = 0.f;
        for (uint32_t i = threadIdx.x * 4; i < K; i += NW * 64 * 4) {
            const float4 v = *reinterpret_cast<const float4 *>(xz + i), wv = *reinterpret_cast<const float4 *>(a.norm_w + i);
            s += (v.x + v.y) + (v.z + v.w);
            *reinterpret_cast<float4 *>(xs + wide_xs_offset(i)) = make_float4(v.x * wv.x, v.y * wv.y, v.z * wv.z, v.w * wv.w);
        }
        const float mean = wide_block_sum(s, stat, w, lane) / (float)K;
        float qd = 0.f;
        for (uint32_t i = threadIdx.x * 4; i < K; i += NW * 64 * 4) {
            const float4 v = *reinterpret_cast<const float4 *>(xz + i);   // second look at x: cache hits
            const float c0 = v.x - mean, c1 = v.y - mean, c2 = v.z - mean, c3 = v.w - mean;
            qd = fmaf(c0, c0, qd); qd = fmaf(c1, c1, qd); qd = fmaf(c2, c2, qd); qd = fmaf(c3, c3, qd);
        }
        inv = rsqrtf(wide_block_sum(qd, stat + 16, w, lane) / (float)K);   // its barrier also publishes xs
    } else {
        for (uint32_t i = threadIdx.x * 4; i < K; i += NW * 64 * 4) *reinterpret_cast<float4 *>(xs + wide_xs_offset(i)) = *reinterpret_cast<const float4 *>(xz + i);
        wide_lds_barrier();
    }
    float xr[32], xsum = 0.f;
    {
        const uint32_t blk = lane_ok ? blk_col : 0;
        const float4 *src = reinterpret_cast<const float4 *>(xs + (size_t)blk * 32);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float4 v = src[(j + blk) & 7];
            if (!lane_ok) v = make_float4(0.f, 0.f, 0.f, 0.f);
            xr[4 * j] = v.x; xr[4 * j + 1] = v.y; xr[4 * j + 2] = v.z; xr[4 * j + 3] = v.w;
            xsum += (v.x + v.y) + (v.z + v.w);
        }
    }

    // ---- rows, DEPTH per turn of the queue, reduced four at a time ---------------------------------------------------
    const uint32_t per_set_q = (per_set + DEPTH - 1) / DEPTH * DEPTH;
    for (uint32_t i0 = 0; i0 < per_set_q; i0 += DEPTH) {
#pragma unroll
        for (int g = 0; g < DEPTH; g += 4) {
            float p[NMAT][4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
#pragma unroll
                for (int mi = 0; mi < NMAT; mi++) p[mi][j] = wide_dot<QT, SF32>(q[mi][g + j], xr, xsum);
                fetch(g + j, i0 + g + j + DEPTH);
            }
#pragma unroll
            for (int mi = 0; mi < NMAT; mi++) {
                const float s = quad_partials_sum(p[mi][0], p[mi][1], p[mi][2], p[mi][3]);
                const uint32_t i = i0 + g + quad_partial_of_lane(lane);
                if (active && (lane & 15) == 0 && i < per_set) red[(((size_t)rset * per_set + i) * NMAT + mi) * NS + slab] = s;
            }
        }
    }
    wide_lds_barrier();

    // ---- combine the slabs, write ---------------------------------------------------------------------------------------
    for (uint32_t r = threadIdx.x; r < n_rows; r += NW * 64) {
        // row r of the workgroup lives in row set r / per_set at index r % per_set: the same slot as above
        float v[NMAT];
#pragma unroll
        for (int mi = 0; mi < NMAT; mi++) {
            float t = 0.f;
            for (int s = 0; s < NS; s++) t += red[((size_t)r * NMAT + mi) * NS + s];
            v[mi] = t;
        }
#pragma unroll
        for (int mi = 0; mi < NMAT; mi++) v[mi] *= inv;
        float *o = a.out + (size_t)z * N + row0 + r;
        if constexpr (MODE == kGemvStore) {
            *o = v[0];
            if (a.cache) {
                const uint32_t row = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add + z;
                if (row < a.backlog) a.cache[(size_t)row * N + row0 + r] = float_to_half_bits(v[0]);
            }
        } else if constexpr (MODE == kGemvAdd) {
            *o += v[0];
        } else {
            *o = v[0] * v[NMAT - 1] / (__expf(-v[NMAT - 1]) + 1.f);
        }
    }
}

template <int QT, int MODE, bool SF32 = false>
__global__ __launch_bounds__(kWideWaves * 64) void gemv_wide_kernel(GemvArgs a, uint32_t rows_per_wg)
{
    __shared__ __attribute__((aligned(16))) float xs[kWideMaxK];
    __shared__ float stat[32];
    extern __shared__ float red[];       // [rows_per_wg rounded up to 4*NR][NMAT][NS]
    gemv_wide_body<QT, MODE, SF32>(a, rows_per_wg, blockIdx.y, xs, red, stat);
}

// Three matrices with the same input vector in one launch (Wq, Wk, Wv of a layer): blockIdx.y selects the matrix.
struct GemvArgs3 {
    GemvArgs m[3];
};
template <int QT, bool SF32 = false>
__global__ __launch_bounds__(kWideWaves * 64) void gemv_wide3_kernel(GemvArgs3 a, uint32_t rows_per_wg)
{
    __shared__ __attribute__((aligned(16))) float xs[kWideMaxK];
    __shared__ float stat[32];
    extern __shared__ float red[];
    gemv_wide_body<QT, kGemvStore, SF32>(a.m[blockIdx.y], rows_per_wg, 0, xs, red, stat);
}

}  // namespace lv
