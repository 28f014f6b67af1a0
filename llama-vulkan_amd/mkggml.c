/*
 * mkggml — deterministic synthetic GGJT (v3) model writer.
 *
 * Produces LLaMA-shaped model files in the on-disk format the reference parses
 * (ggml_file.cpp:17-122: 9-word header, vocab records, tensor records whose payload
 * starts on a 32-byte file offset) filled from a self-contained RNG (splitmix64 +
 * Box-Muller), so the CPU checker and the HIP path read the very same bytes on any box.
 *
 *   q4_0 block (18 B): fp16 scale |N(0,sigma)|, 16 bytes of uniform 4-bit codes
 *   q8_0 block (34 B): fp16 scale |N(0,sigma)|, 32 int8 codes uniform in [-127,127]
 *   f32 tensors (token embeddings, norm weights): N(0,sigma)
 *
 * Every (tensor, row) has its own RNG stream, so rows are generated in parallel and the
 * bytes do not depend on the thread count.
 *
 * Build: cc -O2 -fopenmp -shared -fPIC mkggml.c -o libmkggml.so -lm   (library)
 *        cc -O2 -fopenmp -DMKGGML_MAIN mkggml.c -o mkggml -lm          (command line tool)
 */
#define _GNU_SOURCE
#include <errno.h>
#include <fcntl.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

enum { MKG_F32 = 0, MKG_Q4_0 = 2, MKG_Q8_0 = 8 };

typedef struct {
    uint32_t vocab, dim, heads, layers, ff, multiple_of;
    uint32_t wtype; /* MKG_Q4_0 or MKG_Q8_0 for the matrices */
    uint64_t seed;
    float sigma;    /* 0.02 in the published configs */
    uint32_t tok_type; /* 0: embedding table in f32 (the published configs); MKG_Q4_0 / MKG_Q8_0: quantised like the matrices,
                          as files converted from real checkpoints have it */
} mkg_config;

/* ---------------- RNG ---------------- */

static inline uint64_t splitmix64(uint64_t *s)
{
    uint64_t z = (*s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

static inline uint64_t mix2(uint64_t a, uint64_t b)
{
    uint64_t s = a ^ (b * 0xd6e8feb86659fd93ull + 0x2545f4914f6cdd1dull);
    splitmix64(&s);
    return splitmix64(&s);
}

/* uniform in (0,1] with 53 bits */
static inline double u01(uint64_t *s) { return ((double)(splitmix64(s) >> 11) + 1.0) * (1.0 / 9007199254740992.0); }

/* two independent N(0,1) draws */
static inline void normal2(uint64_t *s, double *a, double *b)
{
    double r = sqrt(-2.0 * log(u01(s)));
    double t = 6.283185307179586476925286766559 * u01(s);
    *a = r * cos(t);
    *b = r * sin(t);
}

/* IEEE fp32 -> fp16, round to nearest even (inputs here are small positive normals or zero) */
static uint16_t f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mag = x & 0x7fffffffu;
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) return (uint16_t)sign;
    uint32_t e = mag >> 23, m = (mag & 0x7fffffu) | 0x800000u;
    uint32_t shift = (e < 113) ? 126 - e : 13;
    uint32_t kept = m >> shift, rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
    uint32_t out = (e < 113) ? kept : ((e - 113) << 10) + kept;
    return (uint16_t)(sign | out);
}

/* ---------------- tensor fills (exported: the kernel microbenchmarks use them directly) ---------------- */

static void fill_quant_row(uint8_t *dst, uint32_t wtype, uint32_t cols, uint64_t stream, float sigma)
{
    uint64_t s = stream;
    uint32_t nb = cols / 32;
    for (uint32_t b = 0; b < nb; b++) {
        double n0, n1;
        normal2(&s, &n0, &n1);
        uint16_t d = f32_to_f16((float)(fabs(n0) * sigma));
        if (wtype == MKG_Q4_0) {
            uint8_t *blk = dst + (size_t)b * 18;
            memcpy(blk, &d, 2);
            uint64_t r0 = splitmix64(&s), r1 = splitmix64(&s);
            memcpy(blk + 2, &r0, 8);
            memcpy(blk + 10, &r1, 8);
        } else {
            uint8_t *blk = dst + (size_t)b * 34;
            memcpy(blk, &d, 2);
            for (int w = 0; w < 8; w++) {
                uint64_t r = splitmix64(&s);
                for (int j = 0; j < 4; j++) {
                    uint32_t u = (uint32_t)((r >> (16 * j)) & 0xffffu);
                    blk[2 + 4 * w + j] = (uint8_t)(int8_t)((int)((u * 255u) >> 16) - 127);
                }
            }
        }
    }
}

size_t mkg_quant_bytes(uint32_t wtype, uint64_t rows, uint64_t cols)
{
    return (size_t)(rows * (cols / 32) * (wtype == MKG_Q4_0 ? 18 : 34));
}

/* rows x cols quantised matrix in GGML block order; stream id = (seed, tensor_id, row) */
void mkg_fill_quant(void *dst, uint32_t wtype, uint32_t rows, uint32_t cols, uint64_t seed, uint64_t tensor_id, float sigma)
{
    size_t row_bytes = mkg_quant_bytes(wtype, 1, cols);
    uint64_t ts = mix2(seed, tensor_id);
#pragma omp parallel for schedule(static)
    for (uint32_t r = 0; r < rows; r++)
        fill_quant_row((uint8_t *)dst + (size_t)r * row_bytes, wtype, cols, mix2(ts, r), sigma);
}

/* rows x cols fp32 N(0,sigma) */
void mkg_fill_normal(float *dst, uint32_t rows, uint32_t cols, uint64_t seed, uint64_t tensor_id, float sigma)
{
    uint64_t ts = mix2(seed, tensor_id);
#pragma omp parallel for schedule(static)
    for (uint32_t r = 0; r < rows; r++) {
        uint64_t s = mix2(ts, r);
        float *row = dst + (size_t)r * cols;
        uint32_t c = 0;
        for (; c + 1 < cols; c += 2) {
            double a, b;
            normal2(&s, &a, &b);
            row[c] = (float)(a * sigma);
            row[c + 1] = (float)(b * sigma);
        }
        if (c < cols) {
            double a, b;
            normal2(&s, &a, &b);
            row[c] = (float)(a * sigma);
        }
    }
}

/* n token ids uniform in [lo, hi) */
void mkg_fill_tokens(uint32_t *dst, uint32_t n, uint32_t lo, uint32_t hi, uint64_t seed)
{
    uint64_t s = mix2(seed, 0x70726f6d7074ull);
    for (uint32_t i = 0; i < n; i++)
        dst[i] = lo + (uint32_t)(splitmix64(&s) % (uint64_t)(hi - lo));
}

/* ---------------- file layout ---------------- */

/* Vocabulary: 0 <unk>, 1 <s>, 2 </s>, 3..258 the 256 single bytes, then printable filler pieces.
 * score = -(float)id, so lower ids merge first. */
static size_t vocab_piece(uint32_t id, char *buf)
{
    if (id == 0) return (size_t)sprintf(buf, "<unk>");
    if (id == 1) return (size_t)sprintf(buf, "<s>");
    if (id == 2) return (size_t)sprintf(buf, "</s>");
    if (id < 259) {
        buf[0] = (char)(id - 3);
        return 1;
    }
    /* two to four lower-case letters derived from the id: distinct for ids < 259 + 26^2 + 26^3 + 26^4 */
    uint32_t k = id - 259, len = 2, span = 26 * 26;
    while (k >= span) {
        k -= span;
        span *= 26;
        len++;
    }
    for (uint32_t i = 0; i < len; i++) {
        buf[len - 1 - i] = (char)('a' + k % 26);
        k /= 26;
    }
    return len;
}

typedef struct {
    char name[96];
    uint32_t ftype, n_dims, ne0, ne1; /* ne0 = columns (written first), ne1 = rows */
    uint64_t offset, size;
} mkg_tensor;

static uint64_t tensor_payload(uint32_t ftype, uint64_t n)
{
    if (ftype == MKG_F32) return n * 4;
    return (n / 32) * (ftype == MKG_Q4_0 ? 18 : 34);
}

static uint32_t build_table(const mkg_config *c, mkg_tensor **out)
{
    uint32_t n = 3 + 9 * c->layers, k = 0;
    mkg_tensor *t = (mkg_tensor *)calloc(n, sizeof(mkg_tensor));
#define ADD2(fmt, arg, ft, cols, rows) \
    do { snprintf(t[k].name, sizeof t[k].name, fmt, arg); t[k].ftype = ft; t[k].n_dims = 2; t[k].ne0 = cols; t[k].ne1 = rows; k++; } while (0)
#define ADD1(fmt, arg, len) \
    do { snprintf(t[k].name, sizeof t[k].name, fmt, arg); t[k].ftype = MKG_F32; t[k].n_dims = 1; t[k].ne0 = len; t[k].ne1 = 1; k++; } while (0)
    ADD2("tok_embeddings.weight%s", "", c->tok_type ? c->tok_type : MKG_F32, c->dim, c->vocab);
    ADD1("norm.weight%s", "", c->dim);
    ADD2("output.weight%s", "", c->wtype, c->dim, c->vocab);
    for (uint32_t i = 0; i < c->layers; i++) {
        ADD2("layers.%u.attention.wq.weight", i, c->wtype, c->dim, c->dim);
        ADD2("layers.%u.attention.wk.weight", i, c->wtype, c->dim, c->dim);
        ADD2("layers.%u.attention.wv.weight", i, c->wtype, c->dim, c->dim);
        ADD2("layers.%u.attention.wo.weight", i, c->wtype, c->dim, c->dim);
        ADD1("layers.%u.attention_norm.weight", i, c->dim);
        ADD2("layers.%u.feed_forward.w1.weight", i, c->wtype, c->dim, c->ff);
        ADD2("layers.%u.feed_forward.w2.weight", i, c->wtype, c->ff, c->dim);
        ADD2("layers.%u.feed_forward.w3.weight", i, c->wtype, c->dim, c->ff);
        ADD1("layers.%u.ffn_norm.weight", i, c->dim);
    }
#undef ADD1
#undef ADD2
    *out = t;
    return k;
}

static int pwrite_all(int fd, const void *src, size_t n, off_t at)
{
    const uint8_t *p = (const uint8_t *)src;
    while (n) {
        ssize_t k = pwrite(fd, p, n > (1u << 30) ? (1u << 30) : n, at);
        if (k <= 0) return -1;
        p += k; n -= (size_t)k; at += k;
    }
    return 0;
}

/* Writes the model; returns 0 or a negative errno-style code. */
int mkg_write_model(const char *path, const mkg_config *c)
{
    if (!c || c->heads == 0 || c->dim % c->heads || c->dim % 32 || c->ff % 32 || c->vocab < 259 ||
        (c->wtype != MKG_Q4_0 && c->wtype != MKG_Q8_0) || (c->tok_type != 0 && c->tok_type != MKG_Q4_0 && c->tok_type != MKG_Q8_0))
        return -EINVAL;

    /* pass 1: sizes */
    uint64_t cur = 9 * 4;
    char piece[16];
    for (uint32_t id = 0; id < c->vocab; id++)
        cur += 4 + vocab_piece(id, piece) + 4;
    mkg_tensor *tab;
    uint32_t nt = build_table(c, &tab);
    for (uint32_t i = 0; i < nt; i++) {
        cur += 4 * (3 + tab[i].n_dims) + strlen(tab[i].name);
        cur = (cur + 31) & ~(uint64_t)31;
        tab[i].offset = cur;
        tab[i].size = tensor_payload(tab[i].ftype, (uint64_t)tab[i].ne0 * tab[i].ne1);
        cur += tab[i].size;
    }
    uint64_t total = cur;

    int fd = open(path, O_RDWR | O_CREAT | O_TRUNC, 0644);
    if (fd < 0) { free(tab); return -errno; }

    /* pass 2: header, vocab and tensor records go through one small buffer per region; payloads are
     * generated into a reusable anonymous buffer and written with pwrite (far fewer page faults than a
     * shared file mapping). */
    int rc = 0;
    uint64_t head_bytes = tab[0].offset;
    uint64_t max_payload = 0;
    for (uint32_t i = 0; i < nt; i++)
        if (tab[i].size > max_payload) max_payload = tab[i].size;
    uint8_t *buf = (uint8_t *)calloc(1, head_bytes > max_payload ? head_bytes : max_payload);
    if (!buf) { close(fd); free(tab); return -ENOMEM; }

    uint32_t hdr[9] = { 0x67676a74u, 3, c->vocab, c->dim, c->multiple_of ? c->multiple_of : 256, c->heads, c->layers,
                        c->dim / c->heads, c->wtype == MKG_Q4_0 ? 2u : 7u };
    memcpy(buf, hdr, sizeof hdr);
    uint64_t w = sizeof hdr;
    for (uint32_t id = 0; id < c->vocab; id++) {
        uint32_t len = (uint32_t)vocab_piece(id, piece);
        float score = -(float)id;
        memcpy(buf + w, &len, 4); w += 4;
        memcpy(buf + w, piece, len); w += len;
        memcpy(buf + w, &score, 4); w += 4;
    }
    uint64_t region_start = 0; /* file offset buf[0] corresponds to */
    float sigma = c->sigma > 0 ? c->sigma : 0.02f;
    for (uint32_t i = 0; i < nt && rc == 0; i++) {
        /* record i (+ zero padding up to the payload) sits in buf at [w - region_start, ...) */
        uint8_t *p = buf + (w - region_start);
        uint32_t name_len = (uint32_t)strlen(tab[i].name);
        memcpy(p, &tab[i].n_dims, 4); p += 4;
        memcpy(p, &name_len, 4); p += 4;
        memcpy(p, &tab[i].ftype, 4); p += 4;
        memcpy(p, &tab[i].ne0, 4); p += 4;
        if (tab[i].n_dims == 2) { memcpy(p, &tab[i].ne1, 4); p += 4; }
        memcpy(p, tab[i].name, name_len); p += name_len;
        uint64_t rec_end = w + (uint64_t)(p - (buf + (w - region_start)));
        memset(p, 0, (size_t)(tab[i].offset - rec_end));
        if (pwrite_all(fd, buf, (size_t)(tab[i].offset - region_start), (off_t)region_start)) { rc = -EIO; break; }
        /* payload; stream id of a tensor is its index in the table */
        if (tab[i].ftype == MKG_F32)
            mkg_fill_normal((float *)buf, tab[i].ne1, tab[i].ne0, c->seed, i, sigma);
        else
            mkg_fill_quant(buf, tab[i].ftype, tab[i].ne1, tab[i].ne0, c->seed, i, sigma);
        if (pwrite_all(fd, buf, (size_t)tab[i].size, (off_t)tab[i].offset)) { rc = -EIO; break; }
        w = region_start = tab[i].offset + tab[i].size;
    }
    if (rc == 0 && w != total) rc = -EIO;
    free(buf);
    if (close(fd) < 0 && rc == 0) rc = -errno;
    free(tab);
    return rc;
}

#ifdef MKGGML_MAIN
static void usage(void)
{
    fprintf(stderr,
            "usage: mkggml OUT --preset 7b|13b|tiny [--wtype q4_0|q8_0] [--tok-type f32|q4_0|q8_0] [--seed N]\n"
            "       mkggml OUT --dim D --heads H --layers L --ff F --vocab V [--wtype ...] [--seed N] [--sigma S]\n");
}

int main(int argc, char **argv)
{
    if (argc < 2) { usage(); return 2; }
    mkg_config c = { 32000, 4096, 32, 32, 11008, 256, MKG_Q4_0, 0, 0.02f, 0 };
    for (int i = 2; i < argc; i++) {
        const char *a = argv[i], *v = (i + 1 < argc) ? argv[i + 1] : NULL;
        if (!v) { usage(); return 2; }
        if (!strcmp(a, "--preset")) {
            if (!strcmp(v, "7b")) { c.dim = 4096; c.heads = 32; c.layers = 32; c.ff = 11008; c.vocab = 32000; }
            else if (!strcmp(v, "13b")) { c.dim = 5120; c.heads = 40; c.layers = 40; c.ff = 13824; c.vocab = 32000; }
            else if (!strcmp(v, "tiny")) { c.dim = 256; c.heads = 4; c.layers = 2; c.ff = 704; c.vocab = 512; }
            else { usage(); return 2; }
        } else if (!strcmp(a, "--wtype")) c.wtype = !strcmp(v, "q8_0") ? MKG_Q8_0 : MKG_Q4_0;
        else if (!strcmp(a, "--tok-type")) c.tok_type = !strcmp(v, "q8_0") ? MKG_Q8_0 : !strcmp(v, "q4_0") ? MKG_Q4_0 : 0;
        else if (!strcmp(a, "--seed")) c.seed = strtoull(v, NULL, 0);
        else if (!strcmp(a, "--sigma")) c.sigma = (float)atof(v);
        else if (!strcmp(a, "--dim")) c.dim = (uint32_t)atoi(v);
        else if (!strcmp(a, "--heads")) c.heads = (uint32_t)atoi(v);
        else if (!strcmp(a, "--layers")) c.layers = (uint32_t)atoi(v);
        else if (!strcmp(a, "--ff")) c.ff = (uint32_t)atoi(v);
        else if (!strcmp(a, "--vocab")) c.vocab = (uint32_t)atoi(v);
        else { usage(); return 2; }
        i++;
    }
    int rc = mkg_write_model(argv[1], &c);
    if (rc) fprintf(stderr, "mkggml: %s\n", strerror(-rc));
    return rc ? 1 : 0;
}
#endif
