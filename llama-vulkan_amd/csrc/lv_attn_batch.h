// lv_attn_batch.h — causal attention for a batch of query rows (prompt evaluation): mhsa.comp + softmax.comp +
// kqv_matching.comp with gl_GlobalInvocationID.z > 0.  Query row z sits at cache position pos + z and sees
// positions 0 .. pos + z; all rows of the batch are in the cache before this runs.
//
// Same arithmetic as the one-query kernel: relative rotation per (query, position) pair with the angle
// float(delta) * theta_i (mhsa.comp:45-58), e = exp(score / sqrt(R)) without max subtraction (softmax.comp:33),
// out = sum e * V / sum e (kqv_matching.comp:35-41), V and K read back from the fp16 cache.
//
// One workgroup = one head x 32 query rows; it walks the cache in tiles of 64 positions staged through LDS, so
// a K/V row is fetched once per 32 queries instead of once per query.
#pragma once

#include "lv_kernels.h"

namespace lv {

constexpr int kAttnBatchQ = 32;   // query rows per workgroup
constexpr int kAttnBatchK = 64;   // cache positions per tile

struct AttnBatchArgs {
    float *out;             // [n][H*R]
    const uint16_t *kcache; // [backlog][H*R] fp16
    const uint16_t *vcache;
    const float *q;         // [n][H*R]
    const float2 *trig;     // [backlog][R/2] (cos, sin) of delta * theta_i
    const uint32_t *pos_ptr;
    uint32_t pos_add;       // row z of the batch sits at *pos_ptr + pos_add + z
    uint32_t n, heads, backlog;
};

template <int R>
struct AttnBatchLds {
    float q[kAttnBatchQ][R + 4];                            // +4: rows stay 16-byte aligned and start in different banks
    float k[kAttnBatchK][R + 2];                            // +2: neighbouring positions start in different banks
    uint16_t v[kAttnBatchK][R];
    float2 trig[kAttnBatchQ + kAttnBatchK][R / 2 + 1];      // rows: delta0 .. delta0 + 95
    float p[kAttnBatchQ][kAttnBatchK + 1];
};

template <int R>
__global__ __launch_bounds__(256) void attention_batch_kernel(AttnBatchArgs a)
{
    constexpr int TQ = kAttnBatchQ, TK = kAttnBatchK, DPT = R / 8;   // output dims per thread
    __shared__ __attribute__((aligned(16))) AttnBatchLds<R> l;
    const uint32_t h = blockIdx.x, z0 = blockIdx.y * TQ;
    const uint32_t H = a.heads, D = H * R;
    const uint32_t pos0 = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add;  // cache position of batch row 0
    const int t = threadIdx.x;
    const int zi = t >> 3, sub = t & 7;      // this thread's query row of the tile; its share of keys / dims
    const uint32_t z = z0 + zi;
    const bool zok = z < a.n;
    const uint32_t my_pos = pos0 + z;        // own cache position
    const uint32_t last_pos = min(pos0 + min(z0 + TQ, a.n) - 1, a.backlog - 1);  // newest position any row of the tile sees

    for (int i = t; i < TQ * R / 4; i += 256) {
        const int row = i / (R / 4), c4 = i % (R / 4);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (z0 + row < a.n) v = *reinterpret_cast<const float4 *>(a.q + (size_t)(z0 + row) * D + (size_t)h * R + c4 * 4);
        *reinterpret_cast<float4 *>(&l.q[row][c4 * 4]) = v;
    }

    const float scale = rsqrtf((float)R);
    float acc[DPT];
#pragma unroll
    for (int i = 0; i < DPT; i++) acc[i] = 0.f;
    float den = 0.f;

    for (uint32_t k0 = 0; k0 <= last_pos; k0 += TK) {
        __syncthreads();  // the previous tile is consumed (and l.q is written, first time round)
        // ---- stage K (as fp32), V (fp16) and the rotation rows of this tile --------------------------------
        for (int i = t; i < TK * R / 8; i += 256) {
            const int row = i / (R / 8), c8 = i % (R / 8);
            const uint32_t p = min(k0 + row, a.backlog - 1);
            const uint4 kraw = *reinterpret_cast<const uint4 *>(a.kcache + (size_t)p * D + (size_t)h * R + c8 * 8);
            const uint4 vraw = *reinterpret_cast<const uint4 *>(a.vcache + (size_t)p * D + (size_t)h * R + c8 * 8);
            const uint32_t kw[4] = {kraw.x, kraw.y, kraw.z, kraw.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                l.k[row][c8 * 8 + 2 * j] = half_bits_to_float((uint16_t)(kw[j] & 0xffffu));
                l.k[row][c8 * 8 + 2 * j + 1] = half_bits_to_float((uint16_t)(kw[j] >> 16));
            }
            *reinterpret_cast<uint4 *>(&l.v[row][c8 * 8]) = vraw;
        }
        // delta of (query row zi, tile position kj) = (pos0 + z0 + zi) - (k0 + kj) = base + zi + (TK - 1 - kj), base = pos0 + z0 - k0 - (TK - 1)
        const int base = (int)(pos0 + z0) - (int)k0 - (TK - 1);
        for (int i = t; i < (TQ + TK) * (R / 2); i += 256) {
            const int row = i / (R / 2), c = i % (R / 2);
            const int delta = base + row;
            const int dc = delta < 0 ? 0 : (delta >= (int)a.backlog ? (int)a.backlog - 1 : delta);  // rows of masked pairs are never used
            l.trig[row][c] = a.trig[(size_t)dc * (R / 2) + c];
        }
        __syncthreads();

        // ---- scores: this thread does keys sub, sub + 8, ... of its query row ---------------------------------
#pragma unroll 1
        for (int m = 0; m < TK / 8; m++) {
            const int kj = sub + 8 * m;
            const uint32_t p = k0 + kj;
            float e = 0.f;
            if (zok && p <= my_pos && p < a.backlog) {
                const float2 *tr = l.trig[zi + (TK - 1 - kj)];
                float s = 0.f;
#pragma unroll 8
                for (int i = 0; i < R / 2; i++) {
                    const float2 qq = *reinterpret_cast<const float2 *>(&l.q[zi][2 * i]);
                    const float2 kk = *reinterpret_cast<const float2 *>(&l.k[kj][2 * i]);
                    const float2 cs = tr[i];
                    const float dotp = fmaf(qq.y, kk.y, qq.x * kk.x);
                    const float crs = fmaf(qq.x, kk.y, -(qq.y * kk.x));
                    s = fmaf(cs.x, dotp, s);
                    s = fmaf(cs.y, crs, s);
                }
                e = __expf(s * scale);
            }
            l.p[zi][kj] = e;
            den += e;
        }
        __syncthreads();

        // ---- P.V: this thread owns dims sub*DPT .. +DPT-1 of its query row ------------------------------------
        const uint32_t lim = min((uint32_t)TK, last_pos + 1 - k0);
        for (uint32_t kj = 0; kj < lim; kj++) {
            const float e = l.p[zi][kj];
            const uint16_t *vr = &l.v[kj][sub * DPT];
#pragma unroll
            for (int i = 0; i < DPT; i++) acc[i] = fmaf(e, half_bits_to_float(vr[i]), acc[i]);
        }
    }

    // the 8 threads of a query row hold partial denominators
    den += __shfl_xor(den, 1, kWave);
    den += __shfl_xor(den, 2, kWave);
    den += __shfl_xor(den, 4, kWave);
    if (zok) {
        float *o = a.out + (size_t)z * D + (size_t)h * R + sub * DPT;
#pragma unroll
        for (int i = 0; i < DPT; i++) o[i] = acc[i] / den;
    }
}

}  // namespace lv
