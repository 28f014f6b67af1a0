// lv_attn_batch.h — causal attention for a batch of query rows (prompt evaluation): mhsa.comp + softmax.comp +
// kqv_matching.comp with gl_GlobalInvocationID.z > 0.  Query row z sits at cache position pos + z and sees
// positions 0 .. pos + z; all rows of the batch are in the cache before this runs.
//
// Arithmetic.  mhsa.comp:45-58 rotates every (query, position) pair by the relative angle delta * theta_i:
//     s = sum_i cos(delta theta_i) (qx kx + qy ky) + sin(delta theta_i) (qx ky - qy kx),   delta = pos_q - pos_k.
// That is Re[conj(q') k'] with q' = e^{i pos_q theta} q and k' = e^{i pos_k theta} k: rotating each query row and each
// cache row ONCE by its own position turns the score into a plain dot product.  The rotation angles come from a table of
// cos/sin(p * theta_i) with theta_i rounded to fp32 as the shader's pow() result is and the product taken exactly; the
// shader rounds delta * theta_i to fp32 before its cos/sin, so the two differ by that one rounding of the angle (below
// 1.3e-4 rad at a distance of 2047, far inside the tolerance that GLSL's own cos/sin precision needs).  The one-query
// kernels keep the per-pair form.  Then e = exp(s / sqrt(R)) without max subtraction (softmax.comp:33),
// out = sum e V / sum e (kqv_matching.comp:35-41), K and V read back from the fp16 cache.  Without a running maximum there
// is nothing to rescale: both sums simply accumulate over the tiles.
//
// Matrix cores at fp32 accuracy.  Both products run on the 16-bit MFMAs (sixteen times the rate of the fp32 ones) with
// their fp32 operands cut into 16-bit pieces whose products the MFMA forms exactly and adds in fp32:
//   scores  q' = qh + ql and k' = kh + kl as fp16 pairs (22 bits); qh kh + ql kh + qh kl, the dropped ql kl is 2^-22 of a term;
//   sums    e = e1 + e2 + e3 as bf16 (an exact cut of the 24 bits; bf16 has fp32's range, and e is not bounded by anything
//           smaller) and the fp16 cache value v = v1 + v2 as bf16 (exact: 11 bits in 8 + 3);
//           e1 v1 + e1 v2 + e2 v1 + e2 v2 + e3 v1, the dropped e3 v2 is 2^-24 of a term.
// attention_prepare_kernel writes the four position-only operand planes of a layer once (kh, kl: rotated K, row-major;
// v1, v2: V transposed, positions along a row, the 16 positions of a group in the order the MFMA's k index wants them),
// so that the attention kernel's inner loop has no conversion in it.
//
// One workgroup = one head x 64 query rows, four waves = 2 query tiles x 2 position tiles of 32; the cache is walked in
// tiles of 64 positions.  A tile's four planes (64 KB at R = 128) go to LDS by direct loads one step ahead of their use
// (two buffers, one barrier per step).  The score MFMA is taken transposed (positions x queries), which leaves a lane
// holding 16 positions of ONE query: exactly the A operand of the second product, with no trip through LDS.
// The 16-byte chunks of a plane's rows are permuted in LDS (chunk ^ row bits) so that the 32 lanes of an operand read,
// which walk down the rows at one chunk, spread over the banks.
#pragma once

#include <type_traits>

#include "lv_gemm.h"

namespace lv {

constexpr int kAttnBatchQ = 64;   // query rows per workgroup
constexpr int kAttnBatchK = 64;   // cache positions per tile

typedef __bf16 lv_b8 __attribute__((ext_vector_type(8)));

// the prepared operand planes of one layer
struct AttnPlanes {
    uint16_t *kh, *kl;      // [rows64][H*R] fp16: rotated K, high and low halves (rows64 = backlog rounded up to 64)
    uint16_t *v1, *v2;      // [H*R][rows64] bf16: V transposed, high and low parts; position order within 16: see attn_slot_pos
};

// position (within its group of 16) held by slot i of a transposed V row: slots 0-3 = positions 0-3, 4-7 = 8-11,
// 8-11 = 4-7, 12-15 = 12-15 (bits 2 and 3 swapped).  A lane of the score MFMA's result holds, in registers 8t .. 8t+7,
// positions 16t + {0-3, 8-11} (lanes 0-31) or 16t + {4-7, 12-15} (lanes 32-63): with this order each is one 16-byte chunk.
__host__ __device__ constexpr int attn_slot_pos(int i) { return (i & 3) | ((i & 4) << 1) | ((i & 8) >> 1); }

__host__ __device__ constexpr uint32_t attn_rows64(uint32_t backlog) { return (backlog + 63) / 64 * 64; }
// halfs of one plane
__host__ __device__ constexpr size_t attn_plane_halfs(uint32_t backlog, uint32_t heads, uint32_t rot) { return (size_t)attn_rows64(backlog) * heads * rot; }

struct AttnPrepArgs {
    AttnPlanes pl;
    uint16_t *kcache, *vcache;          // [backlog][H*R] fp16
    const float *kin, *vin;             // or null: the batch's own K and V rows [n][H*R], which this kernel then also appends to the
                                        // cache (copy_to_cache.comp:29-37: rounded to fp16) and uses as rounded
    const float2 *trig_abs;             // [backlog][R/2] (cos, sin) of p * theta_i
    const uint32_t *pos_ptr;
    uint32_t pos_add;                   // row 0 of the batch sits at *pos_ptr + pos_add
    uint32_t n, heads, backlog;
};

// planes of positions 0 .. pos + n - 1 of one layer; grid (heads, tiles of 64 positions), tiles past the last position return.
// Given the batch's fresh K and V rows it is also the cache append of the batch.
template <int R>
__global__ __launch_bounds__(256) void attention_prepare_kernel(AttnPrepArgs a)
{
    constexpr int TK = kAttnBatchK, C8 = R / 8, VS = R + 2;     // VS: row stride of the staged V tile in halfs
    __shared__ uint32_t vs[TK * VS / 2];
    const uint32_t h = blockIdx.x, k0 = blockIdx.y * TK;
    const uint32_t D = a.heads * R, rows64 = attn_rows64(a.backlog);
    const uint32_t pos0 = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add;
    const uint32_t rows = min(pos0 + a.n, a.backlog);           // positions 0 .. rows-1 hold data
    if (k0 >= rows) return;
    const int t = threadIdx.x;
    for (int g = t; g < C8 * TK; g += 256) {
        const int c8 = g % C8, row = g / C8;
        const uint32_t p = k0 + row;
        float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        uint4 vraw = make_uint4(0u, 0u, 0u, 0u);                // rows past the data: zeros, which the masked sums can take
        if (p < rows) {
            const size_t o = (size_t)p * D + (size_t)h * R + c8 * 8;
            uint4 kraw;
            if (a.kin && p >= pos0) {
                const size_t oi = (size_t)(p - pos0) * D + (size_t)h * R + c8 * 8;
                const float4 k0v = *reinterpret_cast<const float4 *>(a.kin + oi), k1v = *reinterpret_cast<const float4 *>(a.kin + oi + 4);
                const float4 v0v = *reinterpret_cast<const float4 *>(a.vin + oi), v1v = *reinterpret_cast<const float4 *>(a.vin + oi + 4);
                auto pack = [](float lo, float hi) { return (uint32_t)float_to_half_bits(lo) | ((uint32_t)float_to_half_bits(hi) << 16); };
                kraw = make_uint4(pack(k0v.x, k0v.y), pack(k0v.z, k0v.w), pack(k1v.x, k1v.y), pack(k1v.z, k1v.w));
                vraw = make_uint4(pack(v0v.x, v0v.y), pack(v0v.z, v0v.w), pack(v1v.x, v1v.y), pack(v1v.z, v1v.w));
                *reinterpret_cast<uint4 *>(a.kcache + o) = kraw;
                *reinterpret_cast<uint4 *>(a.vcache + o) = vraw;
            } else {
                kraw = *reinterpret_cast<const uint4 *>(a.kcache + o);
                vraw = *reinterpret_cast<const uint4 *>(a.vcache + o);
            }
            const float4 cs0 = *reinterpret_cast<const float4 *>(a.trig_abs + (size_t)p * (R / 2) + c8 * 4);
            const float4 cs1 = *reinterpret_cast<const float4 *>(a.trig_abs + (size_t)p * (R / 2) + c8 * 4 + 2);
            const uint32_t kw[4] = {kraw.x, kraw.y, kraw.z, kraw.w};
            const float c[4] = {cs0.x, cs0.z, cs1.x, cs1.z}, s[4] = {cs0.y, cs0.w, cs1.y, cs1.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // e^{i phi} (x + i y) = (x c - y s) + i (x s + y c)
                const float x = half_bits_to_float((uint16_t)(kw[j] & 0xffffu)), y = half_bits_to_float((uint16_t)(kw[j] >> 16));
                f[2 * j] = x * c[j] - y * s[j];
                f[2 * j + 1] = x * s[j] + y * c[j];
            }
        }
        uint4 hi, lo;
        gemm_split8(hi, lo, f);
        const size_t ok = (size_t)p * D + (size_t)h * R + c8 * 8;   // p < rows64: the planes have that many rows
        *reinterpret_cast<uint4 *>(a.pl.kh + ok) = hi;
        *reinterpret_cast<uint4 *>(a.pl.kl + ok) = lo;
        uint32_t *vrow = vs + (row * VS + c8 * 8) / 2;
        vrow[0] = vraw.x; vrow[1] = vraw.y; vrow[2] = vraw.z; vrow[3] = vraw.w;
    }
    __syncthreads();
    const uint16_t *vh = reinterpret_cast<const uint16_t *>(vs);
    for (int g = t; g < R * 8; g += 256) {
        const int c = g % 8, dim = g / 8;                       // chunk c of the tile's row of this dim: slots 8c .. 8c+7
        uint32_t w1[4], w2[4];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            uint32_t b1[2], b2[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int slot = 8 * c + e + u, pos = (slot & ~15) + attn_slot_pos(slot & 15);
                const float v = half_bits_to_float(vh[pos * VS + dim]);
                b1[u] = __float_as_uint(v) & 0xffff0000u;
                b2[u] = __float_as_uint(v - __uint_as_float(b1[u]));    // three bits at most: the cut to bf16 below loses nothing
            }
            w1[e / 2] = (b1[0] >> 16) | b1[1];
            w2[e / 2] = (b2[0] >> 16) | (b2[1] & 0xffff0000u);
        }
        const size_t o = ((size_t)h * R + dim) * rows64 + k0 + 8 * c;
        *reinterpret_cast<uint4 *>(a.pl.v1 + o) = make_uint4(w1[0], w1[1], w1[2], w1[3]);
        *reinterpret_cast<uint4 *>(a.pl.v2 + o) = make_uint4(w2[0], w2[1], w2[2], w2[3]);
    }
}

struct AttnBatchArgs {
    float *out;             // [n][H*R], or null
    uint16_t *xh, *xl;      // or: the result as the two fp16 halves the output projection's GEMM reads (tile order, width Kp,
                            // rows n .. n_pad-1 zero), or null
    AttnPlanes pl;
    const float *q;         // [n][H*R]
    const float2 *trig_abs; // [backlog][R/2] (cos, sin) of p * theta_i
    const uint32_t *pos_ptr;
    uint32_t pos_add;       // row z of the batch sits at *pos_ptr + pos_add + z
    uint32_t n, heads, backlog, Kp;
};

// LDS chunk permutation of the K planes: rows of 2R bytes; eight consecutive rows at one chunk must fall into eight
// different 16-byte columns of the 128-byte bank row
template <int R>
__device__ __forceinline__ int attn_kswz(int row) { return R >= 64 ? (row & 7) : ((row >> 1) & 3); }

// grid (heads, query tiles of 64 over the padded batch); dynamic LDS: 1024 R bytes
template <int R>
__global__ __launch_bounds__(256) void attention_batch_kernel(AttnBatchArgs a)
{
    constexpr int TQ = kAttnBatchQ, TK = kAttnBatchK;
    constexpr int KS = R / 16;                  // MFMA steps of a score tile (16 k each)
    constexpr int DT = R / 32;                  // 32-wide tiles of the head dimension
    constexpr int PLANE = TK * R * 2;           // bytes of one plane of a tile (K: 64 rows of 2R bytes; V: R rows of 128 bytes)
    constexpr int STAGE = 4 * PLANE;            // kh, kl, v1, v2
    constexpr int NI = PLANE / 1024;            // direct loads (1 KB per wave instruction) per plane
    constexpr int XS = R + 4;                   // row stride of the result exchange in floats
    static_assert(2 * TQ * XS * 4 <= 2 * STAGE, "the result exchange reuses the tile buffers");
    extern __shared__ __attribute__((aligned(16))) uint8_t attn_lds[];
    __shared__ float den_s[2][2][32];           // [position tile][query tile][query row]
    // the last query tile walks the most cache tiles: it is dispatched first, so the short ones fill the tail
    const uint32_t h = blockIdx.x, z0 = (gridDim.y - 1 - blockIdx.y) * TQ;
    const uint32_t H = a.heads, D = H * R, rows64 = attn_rows64(a.backlog);
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    if (z0 >= a.n) {        // rows of the padded batch: zero halves
        if (a.xh)
            for (int g = t; g < TQ * (R / 8); g += 256) {
                const size_t o = gemm_x_offset(z0 + g / (R / 8), h * R + (g % (R / 8)) * 8, a.Kp);
                *reinterpret_cast<uint4 *>(a.xh + o) = make_uint4(0u, 0u, 0u, 0u);
                *reinterpret_cast<uint4 *>(a.xl + o) = make_uint4(0u, 0u, 0u, 0u);
            }
        return;
    }
    const uint32_t pos0 = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add;  // cache position of batch row 0
    const int qt = wave & 1, pt = wave >> 1;      // this wave's query tile and position sub-tile
    const int n32 = lane & 31, hh = lane >> 5;
    const uint32_t last_row = min(z0 + TQ, a.n) - 1;                  // last query row of the workgroup
    const uint32_t last_pos = min(pos0 + last_row, a.backlog - 1);    // newest position any of them sees
    const uint32_t steps = last_pos / TK + 1;

    // ---- direct loads of the tile at k0 into buffer s: every wave issues NI / 4 (at least one) per plane ------------------
    const uint8_t *const gkh = reinterpret_cast<const uint8_t *>(a.pl.kh), *const gkl = reinterpret_cast<const uint8_t *>(a.pl.kl);
    const uint8_t *const gv1 = reinterpret_cast<const uint8_t *>(a.pl.v1), *const gv2 = reinterpret_cast<const uint8_t *>(a.pl.v2);
    auto issue = [&](int s, uint32_t k0) {
        uint8_t *buf = attn_lds + s * STAGE;
#pragma unroll
        for (int i0 = 0; i0 < NI; i0 += 4) {
            const int i = i0 + wave;
            if (NI < 4 && i >= NI) break;
            const int byte = 1024 * i + 16 * lane;
            const int row = byte / (2 * R), c = ((byte % (2 * R)) / 16) ^ attn_kswz<R>(row);
            const size_t gk = ((size_t)(k0 + row) * D + (size_t)h * R + c * 8) * 2;
            __builtin_amdgcn_global_load_lds((lv_glb_void *)(gkh + gk), (lv_lds_void *)(buf + 1024 * i), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((lv_glb_void *)(gkl + gk), (lv_lds_void *)(buf + PLANE + 1024 * i), 16, 0, 0);
            const int dim = byte / 128, cv = (lane & 7) ^ (dim & 7);
            const size_t gv = (((size_t)h * R + dim) * rows64 + k0 + 8 * cv) * 2;
            __builtin_amdgcn_global_load_lds((lv_glb_void *)(gv1 + gv), (lv_lds_void *)(buf + 2 * PLANE + 1024 * i), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((lv_glb_void *)(gv2 + gv), (lv_lds_void *)(buf + 3 * PLANE + 1024 * i), 16, 0, 0);
        }
    };
    issue(0, 0);

    // ---- this lane's query operands: row n32 of the wave's tile, rotated to its own position, as fp16 pairs -------------
    // operand j holds components 16 j + 8 hh .. + 7 of q' (pairs 8 j + 4 hh .. + 3)
    lv_h8 qh[KS], ql[KS];
    const uint32_t zq = z0 + 32 * qt + n32;
    const bool zok = zq < a.n;
    {
        const uint32_t pq = min(pos0 + zq, a.backlog - 1);
        const float *qr = a.q + (size_t)(zok ? zq : 0) * D + (size_t)h * R;
        const float2 *tr = a.trig_abs + (size_t)pq * (R / 2);
#pragma unroll
        for (int j = 0; j < KS; j++) {
            const float4 q0 = *reinterpret_cast<const float4 *>(qr + 16 * j + 8 * hh), q1 = *reinterpret_cast<const float4 *>(qr + 16 * j + 8 * hh + 4);
            const float4 c0 = *reinterpret_cast<const float4 *>(tr + 8 * j + 4 * hh), c1 = *reinterpret_cast<const float4 *>(tr + 8 * j + 4 * hh + 2);
            // e^{i phi} (x + i y) = (x c - y s) + i (x s + y c)
            float f[8] = {q0.x * c0.x - q0.y * c0.y, q0.x * c0.y + q0.y * c0.x, q0.z * c0.z - q0.w * c0.w, q0.z * c0.w + q0.w * c0.z,
                          q1.x * c1.x - q1.y * c1.y, q1.x * c1.y + q1.y * c1.x, q1.z * c1.z - q1.w * c1.w, q1.z * c1.w + q1.w * c1.z};
            if (!zok) {
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] = 0.f;
            }
            uint4 hi, lo;
            gemm_split8(hi, lo, f);
            qh[j] = __builtin_bit_cast(lv_h8, hi);
            ql[j] = __builtin_bit_cast(lv_h8, lo);
        }
    }

    const float scale = rsqrtf((float)R);
    lv_f16v acc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[d][r] = 0.f;
    float den = 0.f;      // sum of this lane's probabilities: query row n32, the positions this lane's registers hold
    const uint32_t wave_last = pos0 + min(z0 + 32 * qt + 31, a.n - 1);   // newest position a query of this wave's tile sees
    const uint32_t limit = pos0 + zq;                                     // newest position this lane's query sees

    for (uint32_t it = 0; it < steps; it++) {
        const uint32_t k0 = it * TK;
        // this wave's direct loads of the tile have landed; behind the barrier everyone's have, and the other buffer is consumed
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (it + 1 < steps) issue((it + 1) & 1, k0 + TK);
        if (k0 + 32 * pt > wave_last) continue;       // every pair of this wave's 32 x 32 tile is masked
        const uint8_t *kb = attn_lds + (it & 1) * STAGE, *vb = kb + 2 * PLANE;

        // ---- scores, transposed: S^T = K' Q'^T; rows = positions k0 + 32 pt .., columns = queries ---------------------------
        lv_f16v sc;
#pragma unroll
        for (int r = 0; r < 16; r++) sc[r] = 0.f;
        {
            const int row = 32 * pt + n32;
            const uint8_t *kr = kb + row * 2 * R;
            const int sw = attn_kswz<R>(row);
#pragma unroll
            for (int j = 0; j < KS; j++) {
                const int c = (2 * j + hh) ^ sw;
                const lv_h8 ah = *reinterpret_cast<const lv_h8 *>(kr + c * 16), al = *reinterpret_cast<const lv_h8 *>(kr + PLANE + c * 16);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, ql[j], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, qh[j], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, qh[j], sc, 0, 0, 0);
            }
        }
        // register r of sc: position k0 + 32 pt + 8 (r / 4) + 4 hh + r % 4, query n32 of the wave's tile
        // ---- O += P V, sixteen positions (registers 8t .. 8t+7 of both lane halves) at a time --------------------------------
        // a tile wholly below the diagonal (every query of the wave's 32 sees every position of its 32) needs no masks
        const bool interior = k0 + 32 * pt + 31 <= pos0 + z0 + 32 * qt && z0 + 32 * qt + 31 < a.n && k0 + 32 * pt + 31 < a.backlog;
        auto sums = [&](auto masked) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                uint32_t w1[4], w2[4], w3[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    uint32_t b1[2], b2[2], b3[2];
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        const int r = 8 * tt + e + u;
                        float e0 = __expf(sc[r] * scale);
                        if constexpr (decltype(masked)::value) {
                            const uint32_t p = k0 + 32 * pt + 8 * (r / 4) + 4 * hh + (r % 4);
                            const bool ok = zok && p <= limit && p < a.backlog;
                            e0 = ok ? e0 : 0.f;
                        }
                        den += e0;
                        b1[u] = __float_as_uint(e0) & 0xffff0000u;
                        const float r1 = e0 - __uint_as_float(b1[u]);
                        b2[u] = __float_as_uint(r1) & 0xffff0000u;
                        b3[u] = __float_as_uint(r1 - __uint_as_float(b2[u]));   // eight bits at most are left
                    }
                    w1[e / 2] = (b1[0] >> 16) | b1[1];
                    w2[e / 2] = (b2[0] >> 16) | b2[1];
                    w3[e / 2] = (b3[0] >> 16) | (b3[1] & 0xffff0000u);
                }
                const lv_b8 p1 = __builtin_bit_cast(lv_b8, make_uint4(w1[0], w1[1], w1[2], w1[3]));
                const lv_b8 p2 = __builtin_bit_cast(lv_b8, make_uint4(w2[0], w2[1], w2[2], w2[3]));
                const lv_b8 p3 = __builtin_bit_cast(lv_b8, make_uint4(w3[0], w3[1], w3[2], w3[3]));
#pragma unroll
                for (int d = 0; d < DT; d++) {
                    const int dim = 32 * d + n32, c = (4 * pt + 2 * tt + hh) ^ (dim & 7);
                    const lv_b8 va = *reinterpret_cast<const lv_b8 *>(vb + dim * 128 + c * 16);
                    const lv_b8 vc = *reinterpret_cast<const lv_b8 *>(vb + PLANE + dim * 128 + c * 16);
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(p3, va, acc[d], 0, 0, 0);
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(p2, vc, acc[d], 0, 0, 0);
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(p2, va, acc[d], 0, 0, 0);
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(p1, vc, acc[d], 0, 0, 0);
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(p1, va, acc[d], 0, 0, 0);
                }
            }
        };
        if (interior) sums(std::false_type{});
        else sums(std::true_type{});
    }

    // ---- combine the two position tiles, divide, write -------------------------------------------------------------
    // acc[d][r]: query row 8 (r / 4) + 4 hh + r % 4 of the wave's tile, dim 32 d + n32.  Both position tiles leave their sums in
    // LDS ([position tile][query row of the workgroup][XS]); then a thread takes 8 dims of a row at a time: sum, divide, write.
    den += __shfl_xor(den, 32, kWave);                    // both lane halves: all positions this wave saw, query row n32
    __syncthreads();                                      // every wave is done with the tile buffers
    if (hh == 0) den_s[pt][qt][n32] = den;
    float *xch = reinterpret_cast<float *>(attn_lds) + pt * (TQ * XS);
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) xch[(32 * qt + 8 * (r / 4) + 4 * hh + (r % 4)) * XS + 32 * d + n32] = acc[d][r];
    __syncthreads();
    const float *x0p = reinterpret_cast<const float *>(attn_lds), *x1p = x0p + TQ * XS;
    for (int g = t; g < TQ * (R / 8); g += 256) {
        const int row = g / (R / 8), c8 = g % (R / 8);
        const uint32_t z = z0 + row;
        const bool live = z < a.n;
        const float total = den_s[0][row >> 5][row & 31] + den_s[1][row >> 5][row & 31];
        const float4 a0 = *reinterpret_cast<const float4 *>(&x0p[row * XS + c8 * 8]), a1 = *reinterpret_cast<const float4 *>(&x0p[row * XS + c8 * 8 + 4]);
        const float4 b0 = *reinterpret_cast<const float4 *>(&x1p[row * XS + c8 * 8]), b1 = *reinterpret_cast<const float4 *>(&x1p[row * XS + c8 * 8 + 4]);
        float f[8] = {(a0.x + b0.x) / total, (a0.y + b0.y) / total, (a0.z + b0.z) / total, (a0.w + b0.w) / total,
                      (a1.x + b1.x) / total, (a1.y + b1.y) / total, (a1.z + b1.z) / total, (a1.w + b1.w) / total};
        if (a.out && live) {
            float *o = a.out + (size_t)z * D + (size_t)h * R + c8 * 8;
            *reinterpret_cast<float4 *>(o) = make_float4(f[0], f[1], f[2], f[3]);
            *reinterpret_cast<float4 *>(o + 4) = make_float4(f[4], f[5], f[6], f[7]);
        }
        if (a.xh) {
            if (!live) {
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] = 0.f;
            }
            uint4 hi, lo;
            gemm_split8(hi, lo, f);
            const size_t o = gemm_x_offset(z, h * R + c8 * 8, a.Kp);
            *reinterpret_cast<uint4 *>(a.xh + o) = hi;
            *reinterpret_cast<uint4 *>(a.xl + o) = lo;
        }
    }
}

}  // namespace lv
