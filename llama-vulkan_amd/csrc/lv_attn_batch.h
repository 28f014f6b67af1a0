// lv_attn_batch.h — causal attention for a batch of query rows (prompt evaluation): mhsa.comp + softmax.comp +
// kqv_matching.comp with gl_GlobalInvocationID.z > 0.  Query row z sits at cache position pos + z and sees
// positions 0 .. pos + z; all rows of the batch are in the cache before this runs.
//
// Arithmetic.  mhsa.comp:45-58 rotates every (query, position) pair by the relative angle delta * theta_i:
//     s = sum_i cos(delta theta_i) (qx kx + qy ky) + sin(delta theta_i) (qx ky - qy kx),   delta = pos_q - pos_k.
// That is Re[conj(q') k'] with q' = e^{i pos_q theta} q and k' = e^{i pos_k theta} k: rotating each query row and each
// cache row ONCE by its own position turns the score into a plain dot product, which the matrix cores take (fp32 MFMA:
// products and sums in fp32).  The rotation angles come from a table of cos/sin(p * theta_i) with theta_i rounded to
// fp32 as the shader's pow() result is and the product taken exactly; the shader rounds delta * theta_i to fp32 before
// its cos/sin, so the two differ by that one rounding of the angle (below 1.3e-4 rad at a distance of 2047, far inside
// the tolerance that GLSL's own cos/sin precision needs).  The one-query kernels keep the per-pair form.
// Then e = exp(s / sqrt(R)) without max subtraction (softmax.comp:33), out = sum e V / sum e (kqv_matching.comp:35-41),
// K and V read back from the fp16 cache.  Without a running maximum there is nothing to rescale: both sums simply
// accumulate over the tiles.
//
// One workgroup = one head x 64 query rows, four waves = 2 query tiles x 2 position tiles of 32; the cache is walked
// in tiles of 64 positions staged through LDS (K rotated, as fp32, x and y components apart; V transposed, fp16, even
// and odd positions apart: both so that an MFMA operand is a run of consecutive LDS words per lane; the 8-byte units
// of a V row are permuted so that the stores of the staging spread over the banks).
#pragma once

#include "lv_kernels.h"

namespace lv {

constexpr int kAttnBatchQ = 64;   // query rows per workgroup
constexpr int kAttnBatchK = 64;   // cache positions per tile

struct AttnBatchArgs {
    float *out;             // [n][H*R]
    const uint16_t *kcache; // [backlog][H*R] fp16
    const uint16_t *vcache;
    const float *q;         // [n][H*R]
    const float2 *trig_abs; // [backlog][R/2] (cos, sin) of p * theta_i
    const uint32_t *pos_ptr;
    uint32_t pos_add;       // row z of the batch sits at *pos_ptr + pos_add + z
    uint32_t n, heads, backlog;
};

typedef float lv_f32x16 __attribute__((ext_vector_type(16)));

template <int R>
struct AttnBatchLds {
    static constexpr int KP = R / 2 + 4;     // row stride of kx / ky in floats (16-byte aligned, rows start in different banks)
    static constexpr int VP = kAttnBatchK / 2 + 8;   // row stride of vt in halfs
    static constexpr int PP = 16 + 4;        // row stride of the probability tiles in floats
    float kx[kAttnBatchK][KP], ky[kAttnBatchK][KP];   // rotated K: components 2i and 2i+1 of the pairs
    uint16_t vt[2][R][VP];                   // V transposed: [position parity][dim][position / 2], 8-byte units permuted:
    // unit u (positions / 2 = 4u .. 4u+3) of the row of a dim in group c8 = dim / 8 is stored at unit u ^ (c8 & 7)
    __device__ static constexpr int vt_unit(int u, int c8) { return u ^ (c8 & 7); }
    float ps[4][2][32][PP];                  // per wave: exp(score) [position parity][query row][position / 2]
    float den[2][2][32];                     // [position tile][query tile][query row]
};

template <int R>
__global__ __launch_bounds__(256) void attention_batch_kernel(AttnBatchArgs a)
{
    constexpr int TQ = kAttnBatchQ, TK = kAttnBatchK;
    constexpr int KS = R / 2;     // MFMA steps of a score tile (2 k each)
    constexpr int DT = R / 32;    // 32-wide tiles of the head dimension
    using L = AttnBatchLds<R>;
    __shared__ __attribute__((aligned(16))) L l;
    // the last query tile walks the most cache tiles: it is dispatched first, so the short ones fill the tail
    const uint32_t h = blockIdx.x, z0 = (gridDim.y - 1 - blockIdx.y) * TQ;
    const uint32_t H = a.heads, D = H * R;
    const uint32_t pos0 = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add;  // cache position of batch row 0
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int qt = wave & 1, pt = wave >> 1;      // this wave's query tile and position sub-tile
    const int n32 = lane & 31, hh = lane >> 5;
    const uint32_t last_row = min(z0 + TQ, a.n) - 1;                  // last query row of the workgroup
    const uint32_t last_pos = min(pos0 + last_row, a.backlog - 1);    // newest position any of them sees

    // ---- this lane's query operands: row n32 of the wave's tile, rotated to its own position ------------------
    // operand j of the score MFMAs is component 2j + hh of q' (hh = 0: x of pair j, hh = 1: y of pair j)
    float qf[KS];
    {
        const uint32_t z = z0 + 32 * qt + n32;
        const bool zok = z < a.n;
        const uint32_t pq = min(pos0 + z, a.backlog - 1);
        const float *qr = a.q + (size_t)(zok ? z : 0) * D + (size_t)h * R;
        const float2 *tr = a.trig_abs + (size_t)pq * (R / 2);
#pragma unroll
        for (int j = 0; j < KS; j += 2) {
            const float4 q2 = *reinterpret_cast<const float4 *>(qr + 2 * j);      // pairs j, j + 1
            const float4 cs = *reinterpret_cast<const float4 *>(tr + j);          // (c, s) of pairs j, j + 1
            // e^{i phi} (x + i y) = (x c - y s) + i (x s + y c)
            const float x0 = q2.x * cs.x - q2.y * cs.y, y0 = q2.x * cs.y + q2.y * cs.x;
            const float x1 = q2.z * cs.z - q2.w * cs.w, y1 = q2.z * cs.w + q2.w * cs.z;
            qf[j] = zok ? (hh ? y0 : x0) : 0.f;
            qf[j + 1] = zok ? (hh ? y1 : x1) : 0.f;
        }
    }

    const float scale = rsqrtf((float)R);
    lv_f32x16 acc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[d][r] = 0.f;
    float den = 0.f;      // sum of this lane's probability operands: query row n32, positions of parity hh

    for (uint32_t k0 = 0; k0 <= last_pos; k0 += TK) {
        __syncthreads();  // the previous tile is consumed
        // ---- stage K (rotated, fp32) and V (transposed, fp16) of this tile ------------------------------------------
        // a thread takes eight dims (c8) of four positions of one parity, base + par + 2m: their V halfs are neighbours
        // in the transposed tile and go out as one 8-byte store per dim.  The 8-byte units of a vt row are permuted by
        // the row's c8 (vt_unit), which spreads the stores of a wave's sixteen c8 over the banks.
        for (int g = t; g < (R / 8) * 16; g += 256) {
            const int c8 = g % (R / 8), rg = g / (R / 8), par = rg & 1, base = (rg >> 1) * 8;
            uint4 kraw[4], vraw[4];
            float4 cs0[4], cs1[4];
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const uint32_t p = min(k0 + base + par + 2 * m, a.backlog - 1);
                kraw[m] = *reinterpret_cast<const uint4 *>(a.kcache + (size_t)p * D + (size_t)h * R + c8 * 8);
                vraw[m] = *reinterpret_cast<const uint4 *>(a.vcache + (size_t)p * D + (size_t)h * R + c8 * 8);
                cs0[m] = *reinterpret_cast<const float4 *>(a.trig_abs + (size_t)p * (R / 2) + c8 * 4);
                cs1[m] = *reinterpret_cast<const float4 *>(a.trig_abs + (size_t)p * (R / 2) + c8 * 4 + 2);
            }
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const int row = base + par + 2 * m;
                const uint32_t kw[4] = {kraw[m].x, kraw[m].y, kraw[m].z, kraw[m].w};
                const float c[4] = {cs0[m].x, cs0[m].z, cs1[m].x, cs1[m].z}, s[4] = {cs0[m].y, cs0[m].w, cs1[m].y, cs1[m].w};
                float xr[4], yr[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x = half_bits_to_float((uint16_t)(kw[j] & 0xffffu)), y = half_bits_to_float((uint16_t)(kw[j] >> 16));
                    xr[j] = x * c[j] - y * s[j];
                    yr[j] = x * s[j] + y * c[j];
                }
                *reinterpret_cast<float4 *>(&l.kx[row][c8 * 4]) = make_float4(xr[0], xr[1], xr[2], xr[3]);
                *reinterpret_cast<float4 *>(&l.ky[row][c8 * 4]) = make_float4(yr[0], yr[1], yr[2], yr[3]);
            }
            const uint32_t vw[4][4] = {{vraw[0].x, vraw[0].y, vraw[0].z, vraw[0].w}, {vraw[1].x, vraw[1].y, vraw[1].z, vraw[1].w},
                                       {vraw[2].x, vraw[2].y, vraw[2].z, vraw[2].w}, {vraw[3].x, vraw[3].y, vraw[3].z, vraw[3].w}};
            const int unit = L::vt_unit(rg >> 1, c8);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // dims c8*8 + 2j (low halfs) and + 2j + 1 (high halfs) at positions m = 0..3
                const uint2 lo = make_uint2((vw[0][j] & 0xffffu) | (vw[1][j] << 16), (vw[2][j] & 0xffffu) | (vw[3][j] << 16));
                const uint2 hi = make_uint2((vw[0][j] >> 16) | (vw[1][j] & 0xffff0000u), (vw[2][j] >> 16) | (vw[3][j] & 0xffff0000u));
                *reinterpret_cast<uint2 *>(&l.vt[par][c8 * 8 + 2 * j][unit * 4]) = lo;
                *reinterpret_cast<uint2 *>(&l.vt[par][c8 * 8 + 2 * j + 1][unit * 4]) = hi;
            }
        }
        __syncthreads();

        // ---- scores of (query tile qt) x (positions k0 + 32 pt ..): S = Q' K'^T ----------------------------------------
        lv_f32x16 sc;
#pragma unroll
        for (int r = 0; r < 16; r++) sc[r] = 0.f;
        {
            const float *kr = hh ? &l.ky[32 * pt + n32][0] : &l.kx[32 * pt + n32][0];   // position n32 of the sub-tile
#pragma unroll
            for (int j = 0; j < KS; j += 4) {
                const float4 k4 = *reinterpret_cast<const float4 *>(kr + j);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[j], k4.x, sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[j + 1], k4.y, sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[j + 2], k4.z, sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[j + 3], k4.w, sc, 0, 0, 0);
            }
        }
        // in sc a lane holds position n32 of the sub-tile and query rows i = 8 (r / 4) + 4 hh + r % 4
        {
            const uint32_t p = k0 + 32 * pt + n32;
            float *prow = &l.ps[wave][n32 & 1][0][n32 >> 1];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = 8 * (r / 4) + 4 * hh + (r % 4);
                const uint32_t z = z0 + 32 * qt + i;
                const bool ok = z < a.n && p <= pos0 + z && p < a.backlog;
                prow[i * L::PP] = ok ? __expf(sc[r] * scale) : 0.f;
            }
        }
        // ---- O += P V: the probabilities come back as the A operand (row = query n32, k = position 2j + hh) ------------
        float pf[16];
        {
            const float *pr = &l.ps[wave][hh][n32][0];
#pragma unroll
            for (int j = 0; j < 16; j += 4) {
                const float4 p4 = *reinterpret_cast<const float4 *>(pr + j);
                pf[j] = p4.x; pf[j + 1] = p4.y; pf[j + 2] = p4.z; pf[j + 3] = p4.w;
                den += (p4.x + p4.y) + (p4.z + p4.w);
            }
        }
#pragma unroll
        for (int d = 0; d < DT; d++) {
            // B operand: V[position 32 pt + 2j + hh][dim 32 d + n32], sixteen consecutive halfs of the transposed tile
            const int dim = 32 * d + n32;
            uint32_t vw[8];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint2 v2 = *reinterpret_cast<const uint2 *>(&l.vt[hh][dim][L::vt_unit(4 * pt + u, dim >> 3) * 4]);
                vw[2 * u] = v2.x;
                vw[2 * u + 1] = v2.y;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(pf[2 * j], half_bits_to_float((uint16_t)(vw[j] & 0xffffu)), acc[d], 0, 0, 0);
                acc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(pf[2 * j + 1], half_bits_to_float((uint16_t)(vw[j] >> 16)), acc[d], 0, 0, 0);
            }
        }
    }

    // ---- combine the two position tiles, divide, write -------------------------------------------------------------
    den += __shfl_xor(den, 32, kWave);                    // both parities: all positions this wave saw, query row n32
    if (hh == 0) l.den[pt][qt][n32] = den;
    __syncthreads();                                      // also: every wave is done with kx / ky
    static_assert(sizeof(l.kx) + sizeof(l.ky) >= (size_t)2 * DT * 16 * 64 * sizeof(float) && offsetof(L, ky) == offsetof(L, kx) + sizeof(l.kx),
                  "the exchange area below spans kx and ky");
    float *xch = &l.kx[0][0];                             // reused: [query tile][dim tile][register][lane]
    if (pt == 1) {
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) xch[((qt * DT + d) * 16 + r) * 64 + lane] = acc[d][r];
    }
    __syncthreads();
    if (pt == 0) {
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = 8 * (r / 4) + 4 * hh + (r % 4);
                const uint32_t z = z0 + 32 * qt + i;
                if (z < a.n) {
                    const float total = acc[d][r] + xch[((qt * DT + d) * 16 + r) * 64 + lane];
                    a.out[(size_t)z * D + (size_t)h * R + 32 * d + n32] = total / (l.den[0][qt][i] + l.den[1][qt][i]);
                }
            }
    }
}

}  // namespace lv
