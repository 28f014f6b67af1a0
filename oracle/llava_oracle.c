/*
 * llava_oracle.c — CPU restatement of the reference's decode arithmetic (see llava_oracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path, never the thing measured or shipped.
 *
 * The restatement keeps the reference's arithmetic *structure* (what is rounded where, which
 * partial sums exist, binary-tree reductions over "workers"), not its GPU launch geometry.
 * All sums are fp32 like the shaders'.
 */
#define _GNU_SOURCE
#include "llava_oracle.h"

#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

/* ------------------------------------------------------------------------------------------
 * fp16 conversions
 * ---------------------------------------------------------------------------------------- */

/* llava_buffer.cpp:142-177 (halfToFloat): exact widening, subnormals renormalised, inf/nan kept. */
float orc_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t expo = (h >> 10) & 0x1fu;
    uint32_t frac = h & 0x3ffu;
    uint32_t bits;
    if (expo == 0) {
        if (frac == 0) {
            bits = sign;
        } else {
            uint32_t shifts = 0;
            while ((frac & 0x400u) == 0) {
                frac <<= 1;
                shifts++;
            }
            bits = sign | ((113u - shifts) << 23) | ((frac & 0x3ffu) << 13);
        }
    } else if (expo == 31) {
        bits = sign | 0x7f800000u | (frac << 13);
    } else {
        bits = sign | ((expo + 112u) << 23) | (frac << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* copy_to_cache.comp:35 — `float16_t(x)`.  GLSL leaves the rounding mode to the driver; the oracle
 * uses IEEE round-to-nearest-even, which is what AMD hardware conversions do by default. */
uint16_t orc_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) { /* inf / nan */
        uint32_t payload = (mag > 0x7f800000u) ? (0x200u | ((mag >> 13) & 0x3ffu)) : 0;
        return (uint16_t)(sign | 0x7c00u | payload);
    }
    if (mag >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) /* <= 2^-25 rounds to zero (ties-to-even at exactly 2^-25) */
        return (uint16_t)sign;
    uint32_t e = mag >> 23;
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;
    uint32_t shift, half_e;
    if (e < 113) { /* subnormal half: value = m * 2^(e-150), unit 2^-24 */
        shift = 126 - e; /* 14..24 */
        half_e = 0;
    } else {
        shift = 13;
        half_e = e - 112;
    }
    uint32_t kept = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u)))
        kept++;
    uint32_t out;
    if (half_e == 0)
        out = kept; /* a carry into bit 10 makes the smallest normal: correct encoding */
    else
        out = ((half_e - 1) << 10) + kept; /* kept has the implicit bit at 0x400; carries propagate */
    return (uint16_t)(sign | out);
}

/* ------------------------------------------------------------------------------------------
 * GGJT block formats
 * ---------------------------------------------------------------------------------------- */

/* ggml_file.cpp:162-186 (size_in_file) */
size_t orc_tensor_bytes(uint32_t ftype, uint32_t file_version, uint64_t n)
{
    switch (ftype) {
    case ORC_F32: return n * 4;
    case ORC_F16: return n * 2;
    case ORC_Q4_0: return (n / 32) * (file_version == 1 ? 20 : 18);
    case ORC_Q8_0: return (n / 32) * (file_version == 1 ? 36 : 34);
    default: return 0;
    }
}

static size_t block_stride(uint32_t ftype, uint32_t file_version)
{
    return orc_tensor_bytes(ftype, file_version, 32);
}

/* Integer-valued codes of one block (already offset: q-8 for q4_0, signed q for q8_0) and its scale.
 * llava_buffer.cpp:347-394 (write_f32).  Element order: v3 q4_0 keeps low nibbles for elements 0..15 and
 * high nibbles for 16..31; v1 q4_0 interleaves (2j, 2j+1); q8_0 is in order. */
static void decode_block(const uint8_t *blk, uint32_t ftype, uint32_t file_version, float w[32], float *d)
{
    const uint8_t *qs;
    if (file_version == 1) {
        memcpy(d, blk, 4);
        qs = blk + 4;
    } else {
        uint16_t hd;
        memcpy(&hd, blk, 2);
        *d = orc_half_to_float(hd);
        qs = blk + 2;
    }
    if (ftype == ORC_Q4_0) {
        if (file_version == 1) {
            for (int j = 0; j < 16; j++) {
                w[2 * j] = (float)((int)(qs[j] & 0xf) - 8);
                w[2 * j + 1] = (float)((int)(qs[j] >> 4) - 8);
            }
        } else {
            for (int j = 0; j < 16; j++) {
                w[j] = (float)((int)(qs[j] & 0xf) - 8);
                w[j + 16] = (float)((int)(qs[j] >> 4) - 8);
            }
        }
    } else { /* q8_0 */
        for (int j = 0; j < 32; j++)
            w[j] = (float)(int8_t)qs[j];
    }
}

/* llava_buffer.cpp:339-401 (write_f32): x = float(code) * scale, one rounding. */
int orc_dequant(const void *src, uint32_t ftype, uint32_t file_version, float *dst, uint32_t count)
{
    if (ftype == ORC_F32) {
        memcpy(dst, src, (size_t)count * 4);
        return 0;
    }
    if (ftype == ORC_F16) {
        const uint16_t *h = (const uint16_t *)src;
        for (uint32_t i = 0; i < count; i++)
            dst[i] = orc_half_to_float(h[i]);
        return 0;
    }
    if ((ftype != ORC_Q4_0 && ftype != ORC_Q8_0) || (count % 32) != 0)
        return -1;
    size_t stride = block_stride(ftype, file_version);
    const uint8_t *p = (const uint8_t *)src;
    for (uint32_t b = 0; b < count / 32; b++) {
        float w[32], d;
        decode_block(p + b * stride, ftype, file_version, w, &d);
        for (int j = 0; j < 32; j++)
            dst[b * 32 + j] = w[j] * d;
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * reductions
 * ---------------------------------------------------------------------------------------- */

/* common.glsl:58-92 (local_sum): binary tree, slot i += slot i+half, halving until one is left.
 * n must be a power of two; buf is destroyed. */
static float tree_sum(float *buf, uint32_t n)
{
    for (uint32_t half = n >> 1; half > 0; half >>= 1)
        for (uint32_t i = 0; i < half; i++)
            buf[i] += buf[i + half];
    return buf[0];
}

static uint32_t floor_pow2(uint32_t v)
{
    uint32_t p = 1;
    while ((p << 1) <= v)
        p <<= 1;
    return p;
}

/* llava_session.cpp:357-375: 128 workers for 4096 columns and for the feed-forward width, 32 for 5120.
 * Other widths (tiny test models; the reference refuses them) get the largest power of two that does
 * not exceed min(128, blocks per row). */
static uint32_t default_workers(uint32_t cols)
{
    if (cols == 5120)
        return 32;
    uint32_t nb = cols / 32;
    uint32_t w = floor_pow2(nb < 128 ? nb : 128);
    return w ? w : 1;
}

/* ------------------------------------------------------------------------------------------
 * GEMV family
 * ---------------------------------------------------------------------------------------- */

/* One block's contribution: matmul.glsl:50-58 / matmul_q8.glsl:50-56.  Eight groups of four consecutive
 * elements (one mat4*vec4 each), accumulated in order; integer-valued codes times fp32 activations. */
static inline float block_dot(const float w[32], const float *x)
{
    float acc = 0.f;
    for (int g = 0; g < 8; g++) {
        const float *ww = w + 4 * g, *xx = x + 4 * g;
        float part = ww[0] * xx[0];
        part += ww[1] * xx[1];
        part += ww[2] * xx[2];
        part += ww[3] * xx[3];
        acc += part;
    }
    return acc;
}

/* Row n of W against `batch` activation rows.  worker y owns blocks y, y+Y, ... (matmul.glsl:46-62):
 * worker_sum += block_value * scale; then the tree over workers (matmul.glsl:64).  res[z] receives the sums. */
static void row_dot(const uint8_t *row, uint32_t ftype, uint32_t ver, uint32_t nb, const float *x, uint32_t cols,
                    uint32_t batch, uint32_t workers, float *ws /* batch*workers scratch */, float *res)
{
    size_t stride = block_stride(ftype, ver);
    for (uint32_t i = 0; i < batch * workers; i++)
        ws[i] = 0.f;
    for (uint32_t b = 0; b < nb; b++) {
        float w[32], d;
        decode_block(row + b * stride, ftype, ver, w, &d);
        uint32_t y = b % workers;
        for (uint32_t z = 0; z < batch; z++)
            ws[z * workers + y] += block_dot(w, x + (size_t)z * cols + 32 * b) * d;
    }
    for (uint32_t z = 0; z < batch; z++)
        res[z] = tree_sum(ws + z * workers, workers);
}

static int gemv_args_ok(uint32_t ftype, uint32_t rows, uint32_t cols, uint32_t workers)
{
    if (ftype != ORC_Q4_0 && ftype != ORC_Q8_0)
        return 0;
    if (rows == 0 || cols == 0 || (cols % 32) != 0)
        return 0;
    if (workers & (workers - 1))
        return 0;
    return 1;
}

/* matmul.glsl:41-74, matmul_q8.glsl:41-72; MATMUL_ADD = `outp += result` (matmul.glsl:67-68). */
int orc_gemv(float *out, const void *w, uint32_t ftype, uint32_t ver, uint32_t rows, uint32_t cols, const float *x,
             uint32_t batch, int accumulate, uint32_t workers)
{
    if (workers == 0)
        workers = default_workers(cols);
    if (!gemv_args_ok(ftype, rows, cols, workers))
        return -1;
    uint32_t nb = cols / 32;
    size_t row_bytes = nb * block_stride(ftype, ver);
    const uint8_t *base = (const uint8_t *)w;
#pragma omp parallel
    {
        float *ws = (float *)malloc(sizeof(float) * (size_t)batch * (workers + 1));
        float *res = ws + (size_t)batch * workers;
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < rows; n++) {
            row_dot(base + (size_t)n * row_bytes, ftype, ver, nb, x, cols, batch, workers, ws, res);
            for (uint32_t z = 0; z < batch; z++) {
                if (accumulate)
                    out[(size_t)z * rows + n] += res[z];
                else
                    out[(size_t)z * rows + n] = res[z];
            }
        }
        free(ws);
    }
    return 0;
}

/* matmul_silu_ff.comp:49-97: result1 = W3 x, result2 = W1 x, out = result1*result2/(exp(-result2)+1). */
int orc_gemv_silu(float *out, const void *w3, const void *w1, uint32_t ftype, uint32_t ver, uint32_t rows,
                  uint32_t cols, const float *x, uint32_t batch, uint32_t workers)
{
    if (workers == 0)
        workers = default_workers(cols);
    if (!gemv_args_ok(ftype, rows, cols, workers))
        return -1;
    uint32_t nb = cols / 32;
    size_t row_bytes = nb * block_stride(ftype, ver);
    const uint8_t *b3 = (const uint8_t *)w3, *b1 = (const uint8_t *)w1;
#pragma omp parallel
    {
        float *ws = (float *)malloc(sizeof(float) * (size_t)batch * (workers + 2));
        float *r1 = ws + (size_t)batch * workers;
        float *r2 = r1 + batch;
#pragma omp for schedule(static)
        for (uint32_t n = 0; n < rows; n++) {
            row_dot(b3 + (size_t)n * row_bytes, ftype, ver, nb, x, cols, batch, workers, ws, r1);
            row_dot(b1 + (size_t)n * row_bytes, ftype, ver, nb, x, cols, batch, workers, ws, r2);
            for (uint32_t z = 0; z < batch; z++)
                out[(size_t)z * rows + n] = r1[z] * r2[z] / (expf(-r2[z]) + 1.f);
        }
        free(ws);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * normalisation, cache append, attention
 * ---------------------------------------------------------------------------------------- */

/* normalize.comp:34-64.  NOT textbook RMSNorm: mean = sum(x)/D; var = sum((x-mean)^2)/D;
 * out = x * w * inversesqrt(var).  No epsilon, and x itself is not centred.  `wgs` threads each own
 * ceil(D/4/wgs) consecutive vec4s; both sums go through the full-workgroup tree. */
void orc_normalize(float *out, const float *x, const float *w, uint32_t dim, uint32_t batch, uint32_t wgs)
{
    if (wgs == 0)
        wgs = 1024;
    uint32_t nvec = dim / 4;
    uint32_t managed = (nvec + wgs - 1) / wgs;
    float *part = (float *)malloc(sizeof(float) * wgs);
    for (uint32_t z = 0; z < batch; z++) {
        const float *xr = x + (size_t)z * dim;
        float *outr = out + (size_t)z * dim;
        for (uint32_t i = 0; i < wgs; i++) {
            float acc = 0.f;
            for (uint32_t j = 0; j < managed; j++) {
                uint32_t v = managed * i + j;
                if (v < nvec) {
                    const float *e = xr + 4 * v;
                    acc += ((e[0] + e[1]) + e[2]) + e[3]; /* dot(element, vec4(1)) */
                }
            }
            part[i] = acc;
        }
        float mean = tree_sum(part, wgs) / (float)dim;
        for (uint32_t i = 0; i < wgs; i++) {
            float acc = 0.f;
            for (uint32_t j = 0; j < managed; j++) {
                uint32_t v = managed * i + j;
                if (v < nvec) {
                    const float *e = xr + 4 * v;
                    float c0 = e[0] - mean, c1 = e[1] - mean, c2 = e[2] - mean, c3 = e[3] - mean;
                    acc += ((c0 * c0 + c1 * c1) + c2 * c2) + c3 * c3; /* dot(element, element) */
                }
            }
            part[i] = acc;
        }
        float inv = 1.0f / sqrtf(tree_sum(part, wgs) / (float)dim);
        for (uint32_t i = 0; i < dim; i++)
            outr[i] = (xr[i] * w[i]) * inv;
    }
    free(part);
}

/* copy_to_cache.comp:29-37: cache[(pos+z)*D + i] = float16_t(in[z*D + i]). */
void orc_kv_append(uint16_t *cache, const float *in, uint32_t pos, uint32_t dim, uint32_t batch)
{
    for (uint32_t z = 0; z < batch; z++)
        for (uint32_t i = 0; i < dim; i++)
            cache[(size_t)(pos + z) * dim + i] = orc_float_to_half(in[(size_t)z * dim + i]);
}

/* mhsa.comp:32-60.  The binding called q_cache is the K cache, current_k is the fresh Q.
 * score(p,h) = sum_i  Q_i . ( [[c, s], [-s, c]] K_i ),  c/s = cos/sin(float(pos+z-p) * 10000^(-i/(R/2))),
 * pairs are adjacent elements (2i, 2i+1).  Unscaled.  The shader also fills slots p > pos+z with
 * values the softmax mask discards; the oracle writes 0 there. */
void orc_mhsa(float *scores, const uint16_t *kcache, const float *q, uint32_t pos, uint32_t backlog, uint32_t heads,
              uint32_t rot, uint32_t batch)
{
    uint32_t dim = heads * rot, half = rot / 2;
    float *freq = (float *)malloc(sizeof(float) * half);
    for (uint32_t i = 0; i < half; i++)
        freq[i] = powf(10000.0f, -(float)i / (float)half);
    for (uint32_t z = 0; z < batch; z++) {
        uint32_t cur = pos + z;
        float *sz = scores + (size_t)z * backlog * heads;
#pragma omp parallel for schedule(static)
        for (uint32_t p = 0; p < backlog; p++) {
            for (uint32_t h = 0; h < heads; h++) {
                float result = 0.f;
                if (p <= cur) {
                    const uint16_t *kr = kcache + (size_t)p * dim + (size_t)h * rot;
                    const float *qr = q + (size_t)z * dim + (size_t)h * rot;
                    for (uint32_t i = 0; i < half; i++) {
                        float kx = orc_half_to_float(kr[2 * i]), ky = orc_half_to_float(kr[2 * i + 1]);
                        float d_theta = (float)(cur - p) * freq[i];
                        float ct = cosf(d_theta), st = sinf(d_theta);
                        float rx = ct * kx + st * ky;  /* rot_mat * raw_Q, columns (ct,-st),(st,ct) */
                        float ry = -st * kx + ct * ky;
                        result += qr[2 * i] * rx + qr[2 * i + 1] * ry;
                    }
                }
                sz[(size_t)p * heads + h] = result;
            }
        }
    }
    free(freq);
}

/* softmax.comp:26-44: a = exp(score * inversesqrt(R)); a = 0 where p > pos+z; out = a / tree-sum over the
 * whole backlog.  No max subtraction. */
void orc_softmax(float *scores, uint32_t pos, uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch)
{
    float factor = 1.0f / sqrtf((float)rot);
    float *col = (float *)malloc(sizeof(float) * backlog * 2);
    for (uint32_t z = 0; z < batch; z++) {
        float *sz = scores + (size_t)z * backlog * heads;
        for (uint32_t h = 0; h < heads; h++) {
            for (uint32_t p = 0; p < backlog; p++) {
                float a = expf(sz[(size_t)p * heads + h] * factor);
                if (p > pos + z)
                    a = 0.f;
                col[p] = a;
                col[backlog + p] = a;
            }
            float total = tree_sum(col + backlog, backlog);
            for (uint32_t p = 0; p < backlog; p++)
                sz[(size_t)p * heads + h] = col[p] / total;
        }
    }
    free(col);
}

/* kqv_matching.comp:27-42: out[c] = tree-sum over all backlog slots of float(V[p][c]) * attn[p][c / R]. */
void orc_kqv(float *out, const uint16_t *vcache, const float *attn, uint32_t backlog, uint32_t heads, uint32_t rot,
             uint32_t batch)
{
    uint32_t dim = heads * rot;
    for (uint32_t z = 0; z < batch; z++) {
        const float *az = attn + (size_t)z * backlog * heads;
#pragma omp parallel
        {
            float *col = (float *)malloc(sizeof(float) * backlog);
#pragma omp for schedule(static)
            for (uint32_t c = 0; c < dim; c++) {
                uint32_t h = c / rot;
                for (uint32_t p = 0; p < backlog; p++)
                    col[p] = orc_half_to_float(vcache[(size_t)p * dim + c]) * az[(size_t)p * heads + h];
                out[(size_t)z * dim + c] = tree_sum(col, backlog);
            }
            free(col);
        }
    }
}

/* llava_session.cpp:144-152: index of the first strict maximum. */
uint32_t orc_sample_greedy(const float *logits, uint32_t n)
{
    uint32_t m = 0;
    for (uint32_t t = 0; t < n; t++)
        if (logits[t] > logits[m])
            m = t;
    return m;
}

/* ------------------------------------------------------------------------------------------
 * GGJT file (ggml_file.cpp:17-122): 9-word header, vocab, tensor records with 32-byte aligned payloads.
 * ---------------------------------------------------------------------------------------- */

typedef struct {
    char *name;
    uint32_t ftype, rows, cols;
    uint64_t offset, size;
} orc_tensor;

struct orc_model {
    uint8_t *map;
    size_t map_size;
    orc_hparams hp;
    orc_tensor *tensors;
    uint32_t n_tensors;
};

static int rd_u32(const orc_model *m, size_t *cur, uint32_t *v)
{
    if (*cur + 4 > m->map_size)
        return -1;
    memcpy(v, m->map + *cur, 4);
    *cur += 4;
    return 0;
}

static const orc_tensor *find_tensor(const orc_model *m, const char *name)
{
    for (uint32_t i = 0; i < m->n_tensors; i++)
        if (strcmp(m->tensors[i].name, name) == 0)
            return &m->tensors[i];
    /* ggml_file.cpp:337-344: fall back to "<name>.weight" */
    size_t len = strlen(name);
    for (uint32_t i = 0; i < m->n_tensors; i++) {
        const char *t = m->tensors[i].name;
        if (strlen(t) == len + 7 && memcmp(t, name, len) == 0 && strcmp(t + len, ".weight") == 0)
            return &m->tensors[i];
    }
    return NULL;
}

orc_model *orc_model_open(const char *path)
{
    int fd = open(path, O_RDONLY);
    if (fd < 0)
        return NULL;
    struct stat st;
    if (fstat(fd, &st) < 0 || st.st_size < 36) {
        close(fd);
        return NULL;
    }
    orc_model *m = (orc_model *)calloc(1, sizeof(*m));
    m->map_size = (size_t)st.st_size;
    m->map = (uint8_t *)mmap(NULL, m->map_size, PROT_READ, MAP_SHARED, fd, 0);
    close(fd);
    if (m->map == MAP_FAILED) {
        free(m);
        return NULL;
    }
    size_t cur = 0;
    uint32_t hdr[9];
    for (int i = 0; i < 9; i++)
        rd_u32(m, &cur, &hdr[i]);
    if (hdr[0] != 0x67676a74u || hdr[7] * hdr[5] != hdr[3])
        goto bad;
    m->hp.file_version = hdr[1];
    m->hp.vocab = hdr[2];
    m->hp.dim = hdr[3];
    m->hp.multiple_of = hdr[4];
    m->hp.heads = hdr[5];
    m->hp.layers = hdr[6];
    m->hp.rot = hdr[7];
    m->hp.ftype = hdr[8];
    for (uint32_t i = 0; i < m->hp.vocab; i++) { /* i32 len, bytes, f32 score */
        uint32_t len;
        if (rd_u32(m, &cur, &len) || cur + len + 4 > m->map_size)
            goto bad;
        cur += len + 4;
    }
    uint32_t cap = 0;
    while (cur != m->map_size) { /* the reference loops until the cursor hits EOF exactly */
        uint32_t n_dims, name_len, ftype, ne0, ne1 = 0;
        if (rd_u32(m, &cur, &n_dims) || rd_u32(m, &cur, &name_len) || rd_u32(m, &cur, &ftype))
            goto bad;
        if (n_dims < 1 || n_dims > 2 || rd_u32(m, &cur, &ne0))
            goto bad;
        if (n_dims == 2 && rd_u32(m, &cur, &ne1))
            goto bad;
        if (cur + name_len > m->map_size)
            goto bad;
        if (m->n_tensors == cap) {
            cap = cap ? cap * 2 : 64;
            m->tensors = (orc_tensor *)realloc(m->tensors, cap * sizeof(orc_tensor));
        }
        orc_tensor *t = &m->tensors[m->n_tensors++];
        t->name = (char *)malloc(name_len + 1);
        memcpy(t->name, m->map + cur, name_len);
        t->name[name_len] = 0;
        cur += name_len;
        t->ftype = ftype;
        /* ggml_file.cpp:86-91: 1-D -> (ne0, 1); 2-D -> rows = ne1, cols = ne0 */
        t->rows = (n_dims == 2) ? ne1 : ne0;
        t->cols = (n_dims == 2) ? ne0 : 1;
        t->offset = (cur + 31) & ~(uint64_t)31;
        t->size = orc_tensor_bytes(ftype, m->hp.file_version, (uint64_t)t->rows * t->cols);
        if (!(ftype <= 3 || ftype == 8) || t->offset + t->size > m->map_size)
            goto bad;
        cur = t->offset + t->size;
    }
    m->hp.n_tensors = m->n_tensors;
    {
        const orc_tensor *w1 = find_tensor(m, "layers.0.feed_forward.w1");
        if (!w1)
            goto bad;
        m->hp.ff = w1->rows; /* ggml_file.cpp:64 */
    }
    return m;
bad:
    orc_model_close(m);
    return NULL;
}

void orc_model_close(orc_model *m)
{
    if (!m)
        return;
    for (uint32_t i = 0; i < m->n_tensors; i++)
        free(m->tensors[i].name);
    free(m->tensors);
    if (m->map && m->map != MAP_FAILED)
        munmap(m->map, m->map_size);
    free(m);
}

void orc_model_hparams(const orc_model *m, orc_hparams *out) { *out = m->hp; }

int orc_model_tensor(const orc_model *m, const char *name, uint32_t *ftype, uint64_t *offset, uint32_t *rows,
                     uint32_t *cols, uint64_t *size)
{
    const orc_tensor *t = find_tensor(m, name);
    if (!t)
        return -1;
    if (ftype) *ftype = t->ftype;
    if (offset) *offset = t->offset;
    if (rows) *rows = t->rows;
    if (cols) *cols = t->cols;
    if (size) *size = t->size;
    return 0;
}

const void *orc_model_data(const orc_model *m, uint64_t offset) { return m->map + offset; }

/* ------------------------------------------------------------------------------------------
 * session: llava_session.cpp:197-229 (embed, pos, run) + llava_layer.cpp:39-75 (block) +
 * llava_command_buffer.cpp:29-45 (final norm + output head)
 * ---------------------------------------------------------------------------------------- */

typedef struct {
    const orc_tensor *wq, *wk, *wv, *wo, *w1, *w2, *w3, *attn_norm, *ffn_norm;
} orc_layer;

enum { TR_NORM_IN = 0, TR_POST_ATTN, TR_POST_ATTN_NORM, TR_FF, TR_OUT, TR_ATTN, TR_COUNT };

struct orc_session {
    const orc_model *m;
    uint32_t backlog, pos;
    orc_layer *layers;
    const orc_tensor *tok, *norm, *output;
    uint16_t **kc, **vc; /* per layer [backlog][dim] fp16, zero filled (llava_layer_session_data.cpp:146-147) */
    float **trace;       /* [layers*TR_COUNT] */
};

static const orc_tensor *need(const orc_model *m, const char *fmt, uint32_t layer)
{
    char name[128];
    snprintf(name, sizeof name, fmt, layer);
    return find_tensor(m, name);
}

orc_session *orc_session_new(const orc_model *m, uint32_t backlog)
{
    if (!m || backlog == 0 || (backlog & (backlog - 1)))
        return NULL;
    orc_session *s = (orc_session *)calloc(1, sizeof(*s));
    s->m = m;
    s->backlog = backlog;
    uint32_t L = m->hp.layers, D = m->hp.dim, F = m->hp.ff;
    s->layers = (orc_layer *)calloc(L, sizeof(orc_layer));
    s->kc = (uint16_t **)calloc(L, sizeof(void *));
    s->vc = (uint16_t **)calloc(L, sizeof(void *));
    s->trace = (float **)calloc((size_t)L * TR_COUNT, sizeof(void *));
    int ok = 1;
    for (uint32_t i = 0; i < L; i++) {
        orc_layer *l = &s->layers[i];
        l->wq = need(m, "layers.%u.attention.wq", i);
        l->wk = need(m, "layers.%u.attention.wk", i);
        l->wv = need(m, "layers.%u.attention.wv", i);
        l->wo = need(m, "layers.%u.attention.wo", i);
        l->w1 = need(m, "layers.%u.feed_forward.w1", i);
        l->w2 = need(m, "layers.%u.feed_forward.w2", i);
        l->w3 = need(m, "layers.%u.feed_forward.w3", i);
        l->attn_norm = need(m, "layers.%u.attention_norm", i);
        l->ffn_norm = need(m, "layers.%u.ffn_norm", i);
        if (!l->wq || !l->wk || !l->wv || !l->wo || !l->w1 || !l->w2 || !l->w3 || !l->attn_norm || !l->ffn_norm)
            ok = 0;
        s->kc[i] = (uint16_t *)calloc((size_t)backlog * D, 2);
        s->vc[i] = (uint16_t *)calloc((size_t)backlog * D, 2);
        for (int t = 0; t < TR_COUNT; t++)
            s->trace[i * TR_COUNT + t] = (float *)calloc(t == TR_FF ? F : t == TR_ATTN ? (size_t)backlog * m->hp.heads : D, sizeof(float));
    }
    s->tok = find_tensor(m, "tok_embeddings");
    s->norm = find_tensor(m, "norm");
    s->output = find_tensor(m, "output");
    if (!ok || !s->tok || !s->norm || !s->output || s->norm->ftype != ORC_F32) {
        orc_session_free(s);
        return NULL;
    }
    return s;
}

void orc_session_free(orc_session *s)
{
    if (!s)
        return;
    for (uint32_t i = 0; i < s->m->hp.layers; i++) {
        if (s->kc) free(s->kc[i]);
        if (s->vc) free(s->vc[i]);
        for (int t = 0; t < TR_COUNT; t++)
            if (s->trace) free(s->trace[i * TR_COUNT + t]);
    }
    free(s->kc);
    free(s->vc);
    free(s->trace);
    free(s->layers);
    free(s);
}

uint32_t orc_session_pos(const orc_session *s) { return s->pos; }

/* llava_session.cpp:390-395 (rewind): forget positions >= pos; cache contents stay. */
void orc_session_rewind(orc_session *s, uint32_t pos)
{
    if (pos < s->pos)
        s->pos = pos;
}

const uint16_t *orc_session_kv(const orc_session *s, uint32_t layer, int which)
{
    return which ? s->vc[layer] : s->kc[layer];
}

/* llava_layer_session_data.cpp:174-181 (restore_kv_cache) + llava_session.cpp:586-588: load n rows of one plane
 * and continue from position n (call for every layer and both planes, then orc_session_set_pos). */
int orc_session_kv_load(orc_session *s, uint32_t layer, int which, const uint16_t *rows, uint32_t n)
{
    if (layer >= s->m->hp.layers || n > s->backlog)
        return -1;
    memcpy(which ? s->vc[layer] : s->kc[layer], rows, (size_t)n * s->m->hp.dim * 2);
    return 0;
}

int orc_session_set_pos(orc_session *s, uint32_t pos)
{
    if (pos > s->backlog)
        return -1;
    s->pos = pos;
    return 0;
}

#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
#else
int orc_num_threads(void) { return 1; }
#endif

const float *orc_session_trace(const orc_session *s, uint32_t layer, int which, uint32_t *count)
{
    if (layer >= s->m->hp.layers || which < 0 || which >= TR_COUNT)
        return NULL;
    if (count)
        *count = (which == TR_FF) ? s->m->hp.ff : (which == TR_ATTN) ? s->backlog * s->m->hp.heads : s->m->hp.dim;
    return s->trace[layer * TR_COUNT + which];
}

static const void *tdata(const orc_model *m, const orc_tensor *t) { return m->map + t->offset; }

int orc_session_eval(orc_session *s, const uint32_t *tokens, uint32_t n, float *logits_last, float *logits_all)
{
    const orc_model *m = s->m;
    const uint32_t D = m->hp.dim, F = m->hp.ff, H = m->hp.heads, R = m->hp.rot, V = m->hp.vocab;
    const uint32_t ver = m->hp.file_version, L = s->backlog;
    if (n == 0 || s->pos + n > L) /* llava_session.cpp:214-217 "Token buffer overflow" */
        return -1;
    for (uint32_t i = 0; i < n; i++)
        if (tokens[i] >= V)
            return -2;

    float *x = (float *)malloc(sizeof(float) * n * D);
    float *nrm = (float *)malloc(sizeof(float) * n * D);
    float *q = (float *)malloc(sizeof(float) * n * D);
    float *k = (float *)malloc(sizeof(float) * n * D);
    float *v = (float *)malloc(sizeof(float) * n * D);
    float *vo = (float *)malloc(sizeof(float) * n * D);
    float *ff = (float *)malloc(sizeof(float) * n * F);
    float *att = (float *)malloc(sizeof(float) * (size_t)n * L * H);
    float *logits = (float *)malloc(sizeof(float) * (size_t)n * V);
    int rc = 0;

    /* llava_session.cpp:219-223: dequantise the embedding rows on the host */
    size_t row_bytes = s->tok->size / V;
    for (uint32_t i = 0; i < n; i++)
        orc_dequant((const uint8_t *)tdata(m, s->tok) + (size_t)tokens[i] * row_bytes, s->tok->ftype, ver,
                    x + (size_t)i * D, D);

    const uint32_t pos = s->pos; /* config.token_count = tokens already in the cache (llava_session.cpp:224) */
    const size_t last = (size_t)(n - 1);
    for (uint32_t li = 0; li < m->hp.layers && rc == 0; li++) {
        const orc_layer *l = &s->layers[li];
        float **tr = &s->trace[li * TR_COUNT];
        orc_normalize(nrm, x, (const float *)tdata(m, l->attn_norm), D, n, 0);
        memcpy(tr[TR_NORM_IN], nrm + last * D, sizeof(float) * D);
        rc |= orc_gemv(k, tdata(m, l->wk), l->wk->ftype, ver, D, D, nrm, n, 0, 0);
        rc |= orc_gemv(q, tdata(m, l->wq), l->wq->ftype, ver, D, D, nrm, n, 0, 0);
        rc |= orc_gemv(v, tdata(m, l->wv), l->wv->ftype, ver, D, D, nrm, n, 0, 0);
        orc_kv_append(s->kc[li], k, pos, D, n);
        orc_kv_append(s->vc[li], v, pos, D, n);
        orc_mhsa(att, s->kc[li], q, pos, L, H, R, n);
        orc_softmax(att, pos, L, H, R, n);
        memcpy(tr[TR_ATTN], att + last * L * H, sizeof(float) * L * H); /* attn_result of the last row, [backlog][heads] */
        orc_kqv(vo, s->vc[li], att, L, H, R, n);
        rc |= orc_gemv(x, tdata(m, l->wo), l->wo->ftype, ver, D, D, vo, n, 1, 0);
        memcpy(tr[TR_POST_ATTN], x + last * D, sizeof(float) * D);
        orc_normalize(nrm, x, (const float *)tdata(m, l->ffn_norm), D, n, 0);
        memcpy(tr[TR_POST_ATTN_NORM], nrm + last * D, sizeof(float) * D);
        rc |= orc_gemv_silu(ff, tdata(m, l->w3), tdata(m, l->w1), l->w3->ftype, ver, F, D, nrm, n, 0);
        memcpy(tr[TR_FF], ff + last * F, sizeof(float) * F);
        rc |= orc_gemv(x, tdata(m, l->w2), l->w2->ftype, ver, D, F, ff, n, 1, 0);
        memcpy(tr[TR_OUT], x + last * D, sizeof(float) * D);
    }
    if (rc == 0) {
        orc_normalize(nrm, x, (const float *)tdata(m, s->norm), D, n, 0);
        rc = orc_gemv(logits, tdata(m, s->output), s->output->ftype, ver, V, D, nrm, n, 0, 0);
    }
    if (rc == 0) {
        if (logits_last)
            memcpy(logits_last, logits + last * V, sizeof(float) * V);
        if (logits_all)
            memcpy(logits_all, logits, sizeof(float) * (size_t)n * V);
        s->pos += n;
    }
    free(x); free(nrm); free(q); free(k); free(v); free(vo); free(ff); free(att); free(logits);
    return rc;
}

/* ------------------------------------------------------------------------------------------
 * The yardstick for tolerances: the same step in double precision.
 *
 * Same operations in the same places as orc_session_eval (llava_layer.cpp:39-75, the shaders cited above), but every
 * sum, product, exp, sin and cos in double, so that what is left is the result the formulas define plus the one
 * rounding the reference's data format imposes: cache rows are fp16 (copy_to_cache.comp:35), rounded here once from
 * the double value.  Two fp32 implementations that sum in different orders each stay within some distance of this
 * result; a test that compares both with it can tell reassociation noise from a wrong kernel.  n tokens at positions
 * pos0 .. pos0 + n - 1, logits of the last one; the cache rows 0 .. pos0 - 1 of every layer are the caller's (per-layer
 * pointers to [pos0][dim] fp16 rows, taken as they are), so a long context can be continued from a copy of a cache.
 * ---------------------------------------------------------------------------------------- */
static uint16_t double_to_half(double d)
{
    float f = (float)d;
    if ((double)f != d) { /* make f the round-to-odd value so that the second rounding is the only one that counts */
        uint32_t u;
        memcpy(&u, &f, 4);
        if (fabs((double)f) > fabs(d))
            u -= 1;
        u |= 1u;
        memcpy(&f, &u, 4);
    }
    return orc_float_to_half(f);
}

/* Experiment knob (0 = off, the yardstick proper): every GEMM input row is first quantised block by block (32 elements) to
 * signed integers of this many bits with one scale per block, s = max|x| / (2^(bits-1) - 1), x' = s * rint(x / s) -- what a
 * kernel that multiplies integer codes by integer activations on the int8 matrix cores would feed them (8 bits), everything
 * else staying exact.  The logits' distance from the unquantised run is the price of that kernel, measured without building it. */
static int g_act_bits = 0;
void orc_forward_f64_activation_bits(int bits) { g_act_bits = bits; }

static const double *quantised_rows(const double *x, uint32_t cols, uint32_t n, double **owned)
{
    *owned = NULL;
    if (g_act_bits <= 1 || cols % 32)
        return x;
    double *y = (double *)malloc(sizeof(double) * (size_t)n * cols);
    const double top = (double)((1u << (g_act_bits - 1)) - 1);
    for (size_t b = 0; b < (size_t)n * cols / 32; b++) {
        double mx = 0;
        for (int j = 0; j < 32; j++)
            mx = fmax(mx, fabs(x[b * 32 + j]));
        const double sc = mx / top;
        for (int j = 0; j < 32; j++)
            y[b * 32 + j] = sc > 0 ? sc * rint(x[b * 32 + j] / sc) : 0.0;
    }
    *owned = y;
    return y;
}

/* out[z][r] (+)= sum_k W[r][k] x[z][k] */
static void gemm_f64(double *out, const orc_model *m, const orc_tensor *t, uint32_t rows, uint32_t cols, const double *x_in,
                     uint32_t n, int accumulate)
{
    const uint32_t ver = m->hp.file_version;
    const size_t row_bytes = orc_tensor_bytes(t->ftype, ver, cols);
    double *owned;
    const double *x = quantised_rows(x_in, cols, n, &owned);
#pragma omp parallel
    {
        float *wf = (float *)malloc(sizeof(float) * cols);
        double *wd = (double *)malloc(sizeof(double) * cols);
#pragma omp for schedule(static)
        for (uint32_t r = 0; r < rows; r++) {
            orc_dequant((const uint8_t *)tdata(m, t) + (size_t)r * row_bytes, t->ftype, ver, wf, cols);
            for (uint32_t k = 0; k < cols; k++)
                wd[k] = (double)wf[k];
            for (uint32_t z = 0; z < n; z++) {
                const double *xz = x + (size_t)z * cols;
                double a0 = 0, a1 = 0, a2 = 0, a3 = 0;
                uint32_t k = 0;
                for (; k + 4 <= cols; k += 4) {
                    a0 += wd[k] * xz[k];
                    a1 += wd[k + 1] * xz[k + 1];
                    a2 += wd[k + 2] * xz[k + 2];
                    a3 += wd[k + 3] * xz[k + 3];
                }
                for (; k < cols; k++)
                    a0 += wd[k] * xz[k];
                const double sum = (a0 + a1) + (a2 + a3);
                double *o = out + (size_t)z * rows + r;
                *o = accumulate ? *o + sum : sum;
            }
        }
        free(wf);
        free(wd);
    }
    free(owned);
}

static void normalize_f64(double *out, const double *x, const float *w, uint32_t dim, uint32_t n)
{
    for (uint32_t z = 0; z < n; z++) {
        const double *xr = x + (size_t)z * dim;
        double mean = 0, var = 0;
        for (uint32_t i = 0; i < dim; i++)
            mean += xr[i];
        mean /= dim;
        for (uint32_t i = 0; i < dim; i++)
            var += (xr[i] - mean) * (xr[i] - mean);
        const double inv = 1.0 / sqrt(var / dim); /* normalize.comp:34-64: centred variance, no epsilon, x itself not centred */
        for (uint32_t i = 0; i < dim; i++)
            out[(size_t)z * dim + i] = xr[i] * (double)w[i] * inv;
    }
}

int orc_forward_f64(const orc_model *m, const uint32_t *tokens, uint32_t n, uint32_t pos0, const uint16_t *const *kcache,
                    const uint16_t *const *vcache, double *logits_last)
{
    if (!m || !tokens || !logits_last || n == 0 || (pos0 && (!kcache || !vcache)))
        return -1;
    const uint32_t D = m->hp.dim, F = m->hp.ff, H = m->hp.heads, R = m->hp.rot, V = m->hp.vocab, half = R / 2;
    const uint32_t ver = m->hp.file_version, T = pos0 + n;
    const orc_tensor *tok = find_tensor(m, "tok_embeddings"), *normw = find_tensor(m, "norm"), *outw = find_tensor(m, "output");
    if (!tok || !normw || !outw)
        return -3;
    for (uint32_t i = 0; i < n; i++)
        if (tokens[i] >= V)
            return -2;
    double *x = (double *)malloc(sizeof(double) * n * D), *nrm = (double *)malloc(sizeof(double) * n * D);
    double *q = (double *)malloc(sizeof(double) * n * D), *vo = (double *)malloc(sizeof(double) * n * D);
    double *k = (double *)malloc(sizeof(double) * (size_t)T * D), *v = (double *)malloc(sizeof(double) * (size_t)T * D);
    double *g1 = (double *)malloc(sizeof(double) * n * F), *g3 = (double *)malloc(sizeof(double) * n * F);
    double *freq = (double *)malloc(sizeof(double) * half);
    float *row = (float *)malloc(sizeof(float) * D);
    int rc = 0;
    for (uint32_t i = 0; i < half; i++)
        freq[i] = pow(10000.0, -(double)i / (double)half);
    const size_t row_bytes = tok->size / V;
    for (uint32_t i = 0; i < n; i++) {
        orc_dequant((const uint8_t *)tdata(m, tok) + (size_t)tokens[i] * row_bytes, tok->ftype, ver, row, D);
        for (uint32_t j = 0; j < D; j++)
            x[(size_t)i * D + j] = (double)row[j];
    }
    for (uint32_t li = 0; li < m->hp.layers && rc == 0; li++) {
        const orc_tensor *wq = need(m, "layers.%u.attention.wq", li), *wk = need(m, "layers.%u.attention.wk", li);
        const orc_tensor *wv = need(m, "layers.%u.attention.wv", li), *wo = need(m, "layers.%u.attention.wo", li);
        const orc_tensor *w1 = need(m, "layers.%u.feed_forward.w1", li), *w2 = need(m, "layers.%u.feed_forward.w2", li);
        const orc_tensor *w3 = need(m, "layers.%u.feed_forward.w3", li);
        const orc_tensor *an = need(m, "layers.%u.attention_norm", li), *fn = need(m, "layers.%u.ffn_norm", li);
        if (!wq || !wk || !wv || !wo || !w1 || !w2 || !w3 || !an || !fn) {
            rc = -3;
            break;
        }
        double *knew = k + (size_t)pos0 * D, *vnew = v + (size_t)pos0 * D;
        for (size_t i = 0; i < (size_t)pos0 * D; i++) { /* rows the caller's cache already holds, as they are */
            k[i] = (double)orc_half_to_float(kcache[li][i]);
            v[i] = (double)orc_half_to_float(vcache[li][i]);
        }
        normalize_f64(nrm, x, (const float *)tdata(m, an), D, n);
        gemm_f64(knew, m, wk, D, D, nrm, n, 0);
        gemm_f64(q, m, wq, D, D, nrm, n, 0);
        gemm_f64(vnew, m, wv, D, D, nrm, n, 0);
        for (size_t i = 0; i < (size_t)n * D; i++) { /* the cache keeps fp16 (copy_to_cache.comp:35) */
            knew[i] = (double)orc_half_to_float(double_to_half(knew[i]));
            vnew[i] = (double)orc_half_to_float(double_to_half(vnew[i]));
        }
        /* mhsa.comp:32-60, softmax.comp:26-44, kqv_matching.comp:27-42: row z (position pos0 + z) over the rows p <= pos0 + z */
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
        for (uint32_t z = 0; z < n; z++) {
            for (uint32_t h = 0; h < H; h++) {
                const uint32_t cur = pos0 + z;
                double *a = (double *)malloc(sizeof(double) * (cur + 1));
                const double *qr = q + (size_t)z * D + (size_t)h * R;
                double total = 0;
                for (uint32_t p = 0; p <= cur; p++) {
                    const double *kr = k + (size_t)p * D + (size_t)h * R;
                    double sc = 0;
                    for (uint32_t i = 0; i < half; i++) {
                        const double th = (double)(cur - p) * freq[i], ct = cos(th), st = sin(th);
                        const double rx = ct * kr[2 * i] + st * kr[2 * i + 1], ry = -st * kr[2 * i] + ct * kr[2 * i + 1];
                        sc += qr[2 * i] * rx + qr[2 * i + 1] * ry;
                    }
                    a[p] = exp(sc / sqrt((double)R));
                    total += a[p];
                }
                for (uint32_t c = 0; c < R; c++) {
                    double acc = 0;
                    for (uint32_t p = 0; p <= cur; p++)
                        acc += v[(size_t)p * D + (size_t)h * R + c] * (a[p] / total);
                    vo[(size_t)z * D + (size_t)h * R + c] = acc;
                }
                free(a);
            }
        }
        gemm_f64(x, m, wo, D, D, vo, n, 1);
        normalize_f64(nrm, x, (const float *)tdata(m, fn), D, n);
        gemm_f64(g3, m, w3, F, D, nrm, n, 0);
        gemm_f64(g1, m, w1, F, D, nrm, n, 0);
        for (size_t i = 0; i < (size_t)n * F; i++) /* matmul_silu_ff.comp:96 */
            g3[i] = g3[i] * g1[i] / (exp(-g1[i]) + 1.0);
        gemm_f64(x, m, w2, D, F, g3, n, 1);
    }
    if (rc == 0) {
        normalize_f64(nrm, x + (size_t)(n - 1) * D, (const float *)tdata(m, normw), D, 1);
        gemm_f64(logits_last, m, outw, V, D, nrm, 1, 0);
    }
    free(x); free(nrm); free(q); free(k); free(v); free(vo); free(g1); free(g3); free(freq); free(row);
    return rc;
}
