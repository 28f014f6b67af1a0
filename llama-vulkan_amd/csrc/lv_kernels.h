// lv_kernels.h — the decode-path kernels for gfx950 (wave64).  Included once by lv_api.hip.
//
// Device layout of a quantised matrix W[N][K] (nb = K/32 blocks per row):
//   codes : [N][nb] x 16 B (q4_0) or 32 B (q8_0), the GGML code bytes of the block unchanged
//   scales: [N][nb] x fp16
// i.e. the 18 / 34 byte GGML block split into two aligned streams; the byte count is unchanged.
#pragma once

#include "lv_device.h"

namespace lv {

struct MatView {
    const uint4 *codes;     // 1 (q4_0) or 2 (q8_0) uint4 per block
    const uint16_t *scales; // fp16 bits (file version 3)
    uint32_t rows, cols;
    const float *scales_f32 = nullptr;   // fp32 block scales of a version-1 file (then `scales` is null)
};

// Scale of block b, raw (as loaded) and as a float.  Which plane a matrix has is uniform over a launch; keeping the
// raw word lets a load queue run ahead and convert only when the block is used.
__device__ __forceinline__ uint32_t mat_scale_raw(const MatView &m, uint64_t b)
{
    return m.scales_f32 ? __float_as_uint(m.scales_f32[b]) : (uint32_t)m.scales[b];
}
__device__ __forceinline__ float mat_scale_value(const MatView &m, uint32_t raw)
{
    return m.scales_f32 ? __uint_as_float(raw) : half_bits_to_float((uint16_t)raw);
}
__device__ __forceinline__ float mat_scale(const MatView &m, uint64_t b) { return mat_scale_value(m, mat_scale_raw(m, b)); }

// ---------------------------------------------------------------------------------------------------------
// GGML blocks -> device layout (runs once per tensor at upload; replaces llava_buffer.cpp:226-323)
// ---------------------------------------------------------------------------------------------------------
// Version-1 files (llava_buffer.cpp:66-71, 193-224): an fp32 scale in front of the codes (20 / 36 B blocks), and q4_0
// nibbles interleaved (byte j carries elements 2j and 2j+1, llava_buffer.cpp:351-359) instead of split (j and j+16).
// The codes are brought into the version-3 order, the scales kept as fp32: nothing is rounded.
template <int QT>
__global__ void repack_v1_kernel(const uint8_t *__restrict__ src, uint4 *__restrict__ codes, float *__restrict__ scales, uint64_t n_blocks)
{
    constexpr int kBlockBytes = QT == 4 ? 20 : 36;
    const uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const uint32_t *p = reinterpret_cast<const uint32_t *>(src + b * kBlockBytes);  // blocks are 4-byte aligned
    scales[b] = __uint_as_float(p[0]);
    if constexpr (QT == 4) {
        uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 32; e++) {
            const uint32_t byte = (p[1 + (e >> 3)] >> (8 * ((e >> 1) & 3))) & 0xffu;      // v1: element e in byte e/2
            const uint32_t nib = (e & 1) ? (byte >> 4) : (byte & 0xfu);
            const int j = e & 15, hi = e >> 4;                                           // v3: byte e%16, nibble e/16
            out[j >> 2] |= nib << (8 * (j & 3) + 4 * hi);
        }
        codes[b] = make_uint4(out[0], out[1], out[2], out[3]);
    } else {
        codes[2 * b] = make_uint4(p[1], p[2], p[3], p[4]);
        codes[2 * b + 1] = make_uint4(p[5], p[6], p[7], p[8]);
    }
}

template <int QT>  // 4: q4_0 (18 B blocks), 8: q8_0 (34 B blocks)
__global__ void repack_kernel(const uint8_t *__restrict__ src, uint4 *__restrict__ codes, uint16_t *__restrict__ scales,
                              uint64_t n_blocks)
{
    constexpr int kBlockBytes = QT == 4 ? 18 : 34;
    constexpr int kCodeWords = QT == 4 ? 4 : 8;
    const uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const uint16_t *p = reinterpret_cast<const uint16_t *>(src + b * kBlockBytes);  // blocks are 2-byte aligned
    scales[b] = p[0];
    uint32_t w[kCodeWords];
#pragma unroll
    for (int i = 0; i < kCodeWords; i++) w[i] = (uint32_t)p[1 + 2 * i] | ((uint32_t)p[2 + 2 * i] << 16);
    uint4 *dst = codes + b * (kCodeWords / 4);
    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
    if constexpr (QT == 8) dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
}

// ---------------------------------------------------------------------------------------------------------
// dequantise: x = float(code - 8) * f32(d)  /  float(int8 code) * f32(d)      (llava_buffer.cpp:361-394)
// One thread per block, 32 floats out.  Exact: a <= 8-bit integer times an 11-bit significand.
// ---------------------------------------------------------------------------------------------------------
template <int QT>
__global__ void dequant_kernel(MatView m, uint64_t first_block, uint64_t n_blocks, float *__restrict__ dst)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_blocks) return;
    const uint64_t b = first_block + i;
    const float d = mat_scale(m, b);
    float4 *out = reinterpret_cast<float4 *>(dst + i * 32);
    if constexpr (QT == 4) {
        const uint4 q = m.codes[b];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        float v[32];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t byte = (w[j >> 2] >> (8 * (j & 3))) & 0xffu;
            v[j] = (float)((int)(byte & 0xfu) - 8) * d;
            v[j + 16] = (float)((int)(byte >> 4) - 8) * d;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    } else {
        const uint4 qa = m.codes[2 * b], qb = m.codes[2 * b + 1];
        const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float4 o;
            o.x = (float)(int8_t)(w[j] & 0xffu) * d;
            o.y = (float)(int8_t)((w[j] >> 8) & 0xffu) * d;
            o.z = (float)(int8_t)((w[j] >> 16) & 0xffu) * d;
            o.w = (float)(int8_t)(w[j] >> 24) * d;
            out[j] = o;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Dequant-fused GEMV.  out[z][n] (=|+=) sum_k W[n][k] x[z][k]            (matmul.glsl, matmul_q8.glsl)
//                      out[z][n] = (W3 x)[n] * silu((W1 x)[n])           (matmul_silu_ff.comp)
//
// A workgroup is 4 wavefronts arranged CW (column waves) x 4/CW (row waves).  A lane owns the block columns
// b = (cw + p*CW)*64 + lane, p < P, keeps their 32 activations in registers for the whole kernel, and walks
// RPW rows: per (row, owned block) one 128-bit load of codes (two for q8_0) + one fp16 scale, 32 FMAs on
// codes converted in registers.  Per row the lane partials are summed with DPP row operations, then across
// the CW column waves through LDS.
// ---------------------------------------------------------------------------------------------------------
enum GemvMode { kGemvStore = 0, kGemvAdd = 1, kGemvSilu = 2 };

struct GemvArgs {
    MatView w;       // matrix (W3 for the SiLU form)
    MatView w1;      // second matrix of the SiLU form
    const float *x;  // [batch][K]
    float *out;      // [batch][N]
    // extras of the streaming kernel (all optional):
    const float *norm_w = nullptr;     // x is normalised with these weights first (normalize.comp) instead of by a launch of its own
    uint16_t *cache = nullptr;         // the result is also appended, as fp16, to this K or V plane [backlog][N] (copy_to_cache.comp)
    const uint32_t *pos_ptr = nullptr; // ... at row *pos_ptr + pos_add
    uint32_t pos_add = 0, backlog = 0;
};

template <int QT>
__device__ __forceinline__ float block_partial(const MatView &m, uint64_t blk, const float (&x)[32], float xoff)
{
    const float d = mat_scale(m, blk);
    float s;
    if constexpr (QT == 4) {
        const uint4 q = m.codes[blk];
        s = q4_block_dot(q, x) - 8.f * xoff;
    } else {
        const uint4 qa = m.codes[2 * blk], qb = m.codes[2 * blk + 1];
        s = q8_block_dot(qa, qb, x) - 128.f * xoff;
    }
    return s * d;  // scale applied after the integer-valued block dot, like matmul.glsl:60
}

template <int QT, int MODE, int CW, int P, int RPW>
__global__ __launch_bounds__(256) void gemv_kernel(GemvArgs a)
{
    constexpr int RW = 4 / CW;
    constexpr int NMAT = MODE == kGemvSilu ? 2 : 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cw = wave % CW, rw = wave / CW;
    const uint32_t N = a.w.rows, K = a.w.cols, nb = K / 32;
    const uint32_t z = blockIdx.y;
    const float *xz = a.x + (size_t)z * K;

    float xr[P][32];
    float xsum[P];
    bool owned[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        const uint32_t b = (uint32_t)(cw + p * CW) * 64 + lane;
        owned[p] = b < nb;
        const float4 *src = reinterpret_cast<const float4 *>(xz + (size_t)(owned[p] ? b : 0) * 32);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float4 v = src[j];
            if (!owned[p]) v = make_float4(0.f, 0.f, 0.f, 0.f);
            xr[p][4 * j] = v.x; xr[p][4 * j + 1] = v.y; xr[p][4 * j + 2] = v.z; xr[p][4 * j + 3] = v.w;
            s += (v.x + v.y) + (v.z + v.w);
        }
        xsum[p] = s;
    }

    const uint32_t row0 = (blockIdx.x * RW + rw) * RPW;
    float acc[NMAT][RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const uint32_t n = row0 + r;
        float s0 = 0.f, s1 = 0.f;
        if (n < N) {
#pragma unroll
            for (int p = 0; p < P; p++) {
                if (owned[p]) {
                    const uint64_t blk = (uint64_t)n * nb + (uint32_t)(cw + p * CW) * 64 + lane;
                    s0 += block_partial<QT>(a.w, blk, xr[p], xsum[p]);
                    if constexpr (NMAT == 2) s1 += block_partial<QT>(a.w1, blk, xr[p], xsum[p]);
                }
            }
        }
        acc[0][r] = s0;
        if constexpr (NMAT == 2) acc[1][r] = s1;
    }

    __shared__ float red[NMAT][RW][CW][RPW];
#pragma unroll
    for (int mi = 0; mi < NMAT; mi++)
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const float t = wave_sum(acc[mi][r]);
            if (lane == 0) red[mi][rw][cw][r] = t;
        }
    __syncthreads();

    if (threadIdx.x < RW * RPW) {
        const int orw = threadIdx.x / RPW, r = threadIdx.x % RPW;
        const uint32_t n = (blockIdx.x * RW + orw) * RPW + r;
        if (n < N) {
            float v[NMAT];
#pragma unroll
            for (int mi = 0; mi < NMAT; mi++) {
                float t = 0.f;
#pragma unroll
                for (int c = 0; c < CW; c++) t += red[mi][orw][c][r];
                v[mi] = t;
            }
            float *o = a.out + (size_t)z * N + n;
            if constexpr (MODE == kGemvStore) *o = v[0];
            else if constexpr (MODE == kGemvAdd) *o += v[0];
            else *o = v[0] * v[NMAT - 1] / (__expf(-v[NMAT - 1]) + 1.f);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// normalize (normalize.comp:34-64): mean-centred variance, no epsilon, x itself not centred.
// One 256-thread workgroup per batch row; x is read once into registers (up to 16 values per thread per
// pass of the outer loop), two block reductions.
// ---------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float block_sum_256(float v, float *lds /* >= 4 floats */)
{
    v = wave_sum(v);
    __syncthreads();  // protect lds reuse between consecutive calls
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    return (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

__device__ __forceinline__ float block_max_256(float v, float *lds /* >= 4 floats */)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    __syncthreads();  // protect lds reuse between consecutive calls
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
}

// The row is read once, as 128-bit loads that are all in flight together, and kept in registers for the three passes
// (up to 8192 floats, a multiple of 4); longer or odd rows walk memory three times.
__global__ __launch_bounds__(256) void normalize_kernel(float *__restrict__ out, const float *__restrict__ x,
                                                        const float *__restrict__ w, uint32_t dim)
{
    __shared__ float lds[4];
    const float *xr = x + (size_t)blockIdx.x * dim;
    float *outr = out + (size_t)blockIdx.x * dim;
    if (dim <= 8192 && dim % 4 == 0) {
        constexpr int PER = 8;
        const uint32_t n4 = dim / 4;
        float4 v[PER], wv[PER];
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const uint32_t i = threadIdx.x + j * 256;
            const bool ok = i < n4;
            v[j] = ok ? reinterpret_cast<const float4 *>(xr)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            wv[j] = ok ? reinterpret_cast<const float4 *>(w)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
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
            if (i < n4)
                reinterpret_cast<float4 *>(outr)[i] = make_float4((v[j].x * wv[j].x) * inv, (v[j].y * wv[j].y) * inv, (v[j].z * wv[j].z) * inv,
                                                                  (v[j].w * wv[j].w) * inv);
        }
        return;
    }
    float s = 0.f;
    for (uint32_t i = threadIdx.x; i < dim; i += 256) s += xr[i];
    const float mean = block_sum_256(s, lds) / (float)dim;
    float v = 0.f;
    for (uint32_t i = threadIdx.x; i < dim; i += 256) {
        const float c = xr[i] - mean;
        v = fmaf(c, c, v);
    }
    const float inv = rsqrtf(block_sum_256(v, lds) / (float)dim);
    for (uint32_t i = threadIdx.x; i < dim; i += 256) outr[i] = (xr[i] * w[i]) * inv;
}

// ---------------------------------------------------------------------------------------------------------
// copy_to_cache (copy_to_cache.comp:29-37).  pos comes from device memory so a captured graph can be replayed.
// ---------------------------------------------------------------------------------------------------------
__global__ void kv_append_kernel(uint16_t *__restrict__ cache, const float *__restrict__ in, const uint32_t *pos_ptr,
                                 uint32_t pos_add, uint32_t dim, uint32_t backlog)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t z = blockIdx.y;
    const uint32_t row = (pos_ptr ? *pos_ptr : 0u) + pos_add + z;
    if (i < dim && row < backlog) cache[(size_t)row * dim + i] = float_to_half_bits(in[(size_t)z * dim + i]);
}

// K and V rows of one layer in one launch (blockIdx.z: 0 = K, 1 = V)
__global__ void kv_append2_kernel(uint16_t *__restrict__ kcache, uint16_t *__restrict__ vcache, const float *__restrict__ k_in,
                                  const float *__restrict__ v_in, const uint32_t *pos_ptr, uint32_t pos_add, uint32_t dim, uint32_t backlog)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t z = blockIdx.y;
    const uint32_t row = (pos_ptr ? *pos_ptr : 0u) + pos_add + z;
    uint16_t *cache = blockIdx.z ? vcache : kcache;
    const float *in = blockIdx.z ? v_in : k_in;
    if (i < dim && row < backlog) cache[(size_t)row * dim + i] = float_to_half_bits(in[(size_t)z * dim + i]);
}

// ---------------------------------------------------------------------------------------------------------
// Embedding gather (llava_session.cpp:219-223 does this on the host): x[z] = dequant(table[token[z]]).
// ---------------------------------------------------------------------------------------------------------
__global__ void embed_f32_kernel(float *__restrict__ x, const float *__restrict__ table, const uint32_t *tokens,
                                 uint32_t dim)
{
    const uint32_t z = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < dim) x[(size_t)z * dim + i] = table[(size_t)tokens[z] * dim + i];
}

template <int QT>
__global__ void embed_quant_kernel(float *__restrict__ x, MatView table, const uint32_t *tokens)
{
    const uint32_t z = blockIdx.y;
    const uint32_t nb = table.cols / 32;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;  // block within the row
    if (i >= nb) return;
    const uint64_t b = (uint64_t)tokens[z] * nb + i;
    const float d = mat_scale(table, b);
    float *dst = x + (size_t)z * table.cols + (size_t)i * 32;
    if constexpr (QT == 4) {
        const uint4 q = table.codes[b];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t byte = (w[j >> 2] >> (8 * (j & 3))) & 0xffu;
            dst[j] = (float)((int)(byte & 0xfu) - 8) * d;
            dst[j + 16] = (float)((int)(byte >> 4) - 8) * d;
        }
    } else {
        const uint4 qa = table.codes[2 * b], qb = table.codes[2 * b + 1];
        const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int j = 0; j < 32; j++) dst[j] = (float)(int8_t)((w[j >> 2] >> (8 * (j & 3))) & 0xffu) * d;
    }
}

// ---------------------------------------------------------------------------------------------------------
// Single-query attention over the fp16 K/V cache: mhsa.comp + softmax.comp + kqv_matching.comp in one kernel.
//
//   s(p)   = sum_i Q_i . Rot(-(cur-p) theta_i) K_i(p)        K un-rotated fp16, Q fp32, adjacent pairs
//   e(p)   = exp(s(p) / sqrt(R)) for p <= cur (no max subtraction, like softmax.comp:33)
//   out[c] = sum_p e(p) V(p)[c] / sum_p e(p)
//
// Grid (heads, splits, batch); a workgroup (4 waves) owns positions [split*chunk, +chunk) of one head.
// R/8 lanes share a cache row: each lane loads 16 B (8 halfs = 4 rotation pairs) of K, later of V.
// cos/sin come from a table trig[delta][R/2] built on the host with the reference's fp32 argument rounding.
// Partial numerators/denominators go to `part`; the last workgroup of a head to finish sums them in split
// order (deterministic) and writes the head's output.
// ---------------------------------------------------------------------------------------------------------
struct AttnArgs {
    float *out;             // [batch][H*R]
    const uint16_t *kcache; // [backlog][H*R]
    const uint16_t *vcache;
    const float *q;         // [batch][H*R]
    const float2 *trig;     // [backlog][R/2] (cos, sin) of delta * theta_i
    float *part;            // [batch][H][splits][R+1]
    uint32_t *counters;     // [batch][H], zero before the launch; left zero after
    const uint32_t *pos_ptr;
    uint32_t pos_add;
    uint32_t heads, backlog, chunk, splits;
};

constexpr int kAttnChunkRows = 64;       // cache positions per workgroup (AttnArgs::chunk must be this)

template <int R>
__global__ __launch_bounds__(256) void attention_kernel(AttnArgs a)
{
    constexpr int LPR = R / 8;        // lanes per cache row
    constexpr int RPWV = 64 / LPR;    // rows per wave per load
    constexpr int RPB = 4 * RPWV;     // rows per workgroup per round
    constexpr int ROUNDS = kAttnChunkRows / RPB;
    static_assert(ROUNDS >= 1 && ROUNDS * RPB == kAttnChunkRows, "chunk must be whole rounds");
    const uint32_t h = blockIdx.x, split = blockIdx.y, z = blockIdx.z;
    const uint32_t H = a.heads, D = H * R;
    const uint32_t cur = (a.pos_ptr ? *a.pos_ptr : 0u) + a.pos_add + z;  // this row's own cache position
    const uint32_t n_valid = min(cur + 1, a.backlog);
    const uint32_t n_splits = (n_valid + kAttnChunkRows - 1) / kAttnChunkRows;   // splits that hold any position
    if (split >= n_splits) return;
    const uint32_t p_begin = split * kAttnChunkRows, p_end = min(p_begin + kAttnChunkRows, n_valid);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR;             // which 8 elements of the row
    const int rsel = wave * RPWV + lane / LPR;

    extern __shared__ float lds[];
    float *red = lds;                       // [4][R+1]

    // Every load of the chunk goes out before anything is used: K, V and rotation rows of all rounds, and the query.
    uint4 kraw[ROUNDS], vraw[ROUNDS];
    float4 t0[ROUNDS], t1[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const uint32_t p = p_begin + r * RPB + rsel;
        const uint32_t pc = p < p_end ? p : p_begin;     // a valid row; its weight is forced to 0 below
        kraw[r] = *reinterpret_cast<const uint4 *>(a.kcache + (size_t)pc * D + (size_t)h * R + sub * 8);
        vraw[r] = *reinterpret_cast<const uint4 *>(a.vcache + (size_t)pc * D + (size_t)h * R + sub * 8);
        const float4 *tp = reinterpret_cast<const float4 *>(a.trig + (size_t)(cur - pc) * (R / 2) + sub * 4);
        t0[r] = tp[0];  // (c0,s0,c1,s1)
        t1[r] = tp[1];  // (c2,s2,c3,s3)
    }
    float qv[8];
    {
        const float4 *qp = reinterpret_cast<const float4 *>(a.q + (size_t)z * D + (size_t)h * R + sub * 8);
        const float4 q0 = qp[0], q1 = qp[1];
        qv[0] = q0.x; qv[1] = q0.y; qv[2] = q0.z; qv[3] = q0.w;
        qv[4] = q1.x; qv[5] = q1.y; qv[6] = q1.z; qv[7] = q1.w;
    }
    const float scale = rsqrtf((float)R);

    // A row's weight is computed and used by the same LPR lanes: no exchange through LDS between scores and P.V.
    float den = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const uint32_t p = p_begin + r * RPB + rsel;
        const uint32_t kw[4] = {kraw[r].x, kraw[r].y, kraw[r].z, kraw[r].w};
        const float ct[4] = {t0[r].x, t0[r].z, t1[r].x, t1[r].z}, st[4] = {t0[r].y, t0[r].w, t1[r].y, t1[r].w};
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float kx = half_bits_to_float((uint16_t)(kw[i] & 0xffffu));
            const float ky = half_bits_to_float((uint16_t)(kw[i] >> 16));
            const float qx = qv[2 * i], qy = qv[2 * i + 1];
            const float dotp = fmaf(qy, ky, qx * kx);      // Q.K of the pair
            const float crs = fmaf(qx, ky, -(qy * kx));    // Qx Ky - Qy Kx
            s = fmaf(ct[i], dotp, s);
            s = fmaf(st[i], crs, s);
        }
        s = group_sum<LPR>(s);
        const float e = p < p_end ? __expf(s * scale) : 0.f;
        den += (sub == 0) ? e : 0.f;
        const uint32_t vw[4] = {vraw[r].x, vraw[r].y, vraw[r].z, vraw[r].w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc[2 * i] = fmaf(e, half_bits_to_float((uint16_t)(vw[i] & 0xffffu)), acc[2 * i]);
            acc[2 * i + 1] = fmaf(e, half_bits_to_float((uint16_t)(vw[i] >> 16)), acc[2 * i + 1]);
        }
    }
    // sum over the RPWV row groups of the wave (lanes with equal `sub`), then over the 4 waves via LDS
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] += __shfl_xor(acc[i], off, kWave);
        den += __shfl_xor(den, off, kWave);
    }
    if (lane < LPR) {
#pragma unroll
        for (int i = 0; i < 8; i++) red[wave * (R + 1) + lane * 8 + i] = acc[i];
        if (lane == 0) red[wave * (R + 1) + R] = den;
    }
    __syncthreads();

    float *my_part = a.part + (((size_t)z * H + h) * a.splits + split) * (R + 1);
    if (threadIdx.x <= R) {
        const int c = threadIdx.x;
        const float t = (red[c] + red[(R + 1) + c]) + (red[2 * (R + 1) + c] + red[3 * (R + 1) + c]);
        if (n_splits == 1) {
            red[c] = t;  // finished here: normalise below
        } else {
            // write-through store at device scope: visible to every other workgroup once it is acknowledged
            __hip_atomic_store(reinterpret_cast<uint32_t *>(my_part + c), __float_as_uint(t), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (n_splits == 1) {
        __syncthreads();
        if (threadIdx.x < R) a.out[(size_t)z * D + (size_t)h * R + threadIdx.x] = red[threadIdx.x] / red[R];
        return;
    }

    // ---- cross-workgroup combine: the last split to arrive sums all partials in split order ---------------
    // Ordering without a release fence (which at device scope writes back the whole L2): the partials are
    // write-through stores, the wave waits for their acknowledgement, then the workgroup counts itself in; the
    // last workgroup reads the partials with device-scope loads, which do not hit stale lines.
    // This leans on gfx950 hardware rules that the HIP memory model does not promise (stores are counted by vmcnt, and a
    // write-through store is acknowledged only once every XCD can see it); lv_device.h refuses any other target.  The
    // parity tests run it with 2..32 splits per head.
    __shared__ uint32_t arrived;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) arrived = __hip_atomic_fetch_add(&a.counters[(size_t)z * H + h], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived != n_splits - 1) return;
    const float *hp = a.part + ((size_t)z * H + h) * a.splits * (R + 1);
    if (threadIdx.x <= R) {
        float t = 0.f;
        for (uint32_t s0 = 0; s0 < n_splits; s0 += 8) {      // eight loads in flight, summed in split order
            uint32_t v[8];
#pragma unroll
            for (int j = 0; j < 8; j++)
                v[j] = s0 + j < n_splits ? __hip_atomic_load(reinterpret_cast<const uint32_t *>(hp + (size_t)(s0 + j) * (R + 1) + threadIdx.x),
                                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                         : 0u;
#pragma unroll
            for (int j = 0; j < 8; j++) t += __uint_as_float(v[j]);
        }
        red[threadIdx.x] = t;
    }
    __syncthreads();
    if (threadIdx.x < R) a.out[(size_t)z * D + (size_t)h * R + threadIdx.x] = red[threadIdx.x] / red[R];
    if (threadIdx.x == 0) a.counters[(size_t)z * H + h] = 0u;  // ready for the next launch / graph replay
}

// ---------------------------------------------------------------------------------------------------------
// Record mode only: the attention weights of one query as a buffer, which the fused kernel above never holds
// (mhsa.comp + softmax.comp leave them in attn_result, laid out [backlog][heads]; slots behind the query's position
// hold 0, softmax.comp:33-35).  One workgroup per head; scores with the per-pair rotation of the shader, no max
// subtraction, the sum taken over the workgroup in a fixed order.  Not on the decode path.
// ---------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_weights_kernel(float *__restrict__ out, const uint16_t *__restrict__ kcache,
                                                           const float *__restrict__ q, const float2 *__restrict__ trig,
                                                           const uint32_t *pos_ptr, uint32_t pos_add, uint32_t heads, uint32_t rot,
                                                           uint32_t backlog)
{
    __shared__ float red[4];
    const uint32_t h = blockIdx.x, half = rot / 2, dim = heads * rot;
    const uint32_t cur = *pos_ptr + pos_add;
    const float factor = 1.0f / sqrtf((float)rot);
    const float *qr = q + (size_t)h * rot;
    float sum = 0.f;
    for (uint32_t p = threadIdx.x; p < backlog; p += 256) {
        float e = 0.f;
        if (p <= cur) {
            const uint16_t *kr = kcache + (size_t)p * dim + (size_t)h * rot;
            const float2 *t = trig + (size_t)(cur - p) * half;
            float score = 0.f;
            for (uint32_t i = 0; i < half; i++) {
                const float kx = half_bits_to_float(kr[2 * i]), ky = half_bits_to_float(kr[2 * i + 1]);
                const float2 cs = t[i];
                const float rx = cs.x * kx + cs.y * ky, ry = -cs.y * kx + cs.x * ky;
                score += qr[2 * i] * rx + qr[2 * i + 1] * ry;
            }
            e = expf(score * factor);
        }
        out[(size_t)p * heads + h] = e;       // un-normalised for now; this thread re-reads its own slots below
        sum += e;
    }
    for (int off = 32; off; off >>= 1) sum += __shfl_xor(sum, off);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    for (uint32_t p = threadIdx.x; p < backlog; p += 256) out[(size_t)p * heads + h] /= total;
}

// ---------------------------------------------------------------------------------------------------------
// Greedy pick (llava_session.cpp:144-152): index of the first strict maximum.  One workgroup.
// ---------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ logits, uint32_t n, uint32_t *out)
{
    __shared__ float bv[1024];
    __shared__ uint32_t bi[1024];
    float best = -INFINITY;
    uint32_t idx = 0xffffffffu;
    for (uint32_t i = threadIdx.x; i < n; i += 1024) {
        const float v = logits[i];
        if (idx == 0xffffffffu || v > best) { best = v; idx = i; }
    }
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = idx;
    __syncthreads();
    for (uint32_t half = 512; half > 0; half >>= 1) {
        if (threadIdx.x < half) {
            const float ov = bv[threadIdx.x + half];
            const uint32_t oi = bi[threadIdx.x + half];
            const float mv = bv[threadIdx.x];
            const uint32_t mi = bi[threadIdx.x];
            // keep the larger value; on equal values (or NaN-free ties) the lower index
            const bool take = (oi != 0xffffffffu) && (mi == 0xffffffffu || ov > mv || (ov == mv && oi < mi));
            if (take) { bv[threadIdx.x] = ov; bi[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = bi[0] == 0xffffffffu ? 0u : bi[0];
}

}  // namespace lv
