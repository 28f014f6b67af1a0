/*
 * llava_oracle.h — CPU restatement of the reference's per-token decode arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may include, link or
 * call this file: only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg use it, and only as the checker.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference tree).  The reference has no tests and no golden vectors, so
 * each function below is pinned by the independent checks in
 * tests/test_oracle_*.py (numpy float16 on all 65 536 half patterns,
 * exhaustive (scale, code) dequant products, fp64 dot products, textbook RoPE,
 * scipy softmax, numpy std, brute force on tiny inputs).
 *
 * Pin status per function:
 *   orc_half_to_float, orc_float_to_half, orc_dequant ......... pinned (exhaustive)
 *   orc_gemv, orc_gemv_silu ................................... pinned (fp64 brute force + special cases)
 *   orc_normalize ............................................. pinned (closed form, non-zero-mean case)
 *   orc_kv_append ............................................. pinned (numpy astype(float16), indexing)
 *   orc_mhsa, orc_softmax, orc_kqv ............................ pinned (textbook RoPE/softmax, one-hot cases)
 *   orc_session_eval (whole step) ............................. pinned by composition + prefill==decode
 *                                                               self-consistency; token identity against
 *                                                               a run of the Vulkan binary: parity unpinned
 *   orc_sample_greedy ......................................... pinned (first strict max by construction)
 *   orc_forward_f64 (double-precision yardstick) .............. pinned (independent numpy fp64 forward pass)
 */
#ifndef LLAVA_ORACLE_H
#define LLAVA_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q4_0 = 2, ORC_Q8_0 = 8 };

/* fp16 <-> fp32 */
float    orc_half_to_float(uint16_t h);
uint16_t orc_float_to_half(float f);

/* bytes one tensor of rows*cols elements occupies in a GGJT file */
size_t orc_tensor_bytes(uint32_t ftype, uint32_t file_version, uint64_t n_elements);

/* dequantise `count` consecutive elements (count % 32 == 0 for quantised types) */
int orc_dequant(const void *src, uint32_t ftype, uint32_t file_version, float *dst, uint32_t count);

/* out[n] (=|+=) sum_k W[n][k] x[k];  `workers` = how many partial sums per row the reference keeps
 * before its binary tree (0 = pick the reference's rule for this column count). */
int orc_gemv(float *out, const void *w, uint32_t ftype, uint32_t file_version, uint32_t rows, uint32_t cols,
             const float *x, uint32_t batch, int accumulate, uint32_t workers);
/* out[n] = (W3 x)[n] * silu((W1 x)[n]) */
int orc_gemv_silu(float *out, const void *w3, const void *w1, uint32_t ftype, uint32_t file_version, uint32_t rows,
                  uint32_t cols, const float *x, uint32_t batch, uint32_t workers);

void orc_normalize(float *out, const float *x, const float *w, uint32_t dim, uint32_t batch, uint32_t wgs);
void orc_kv_append(uint16_t *cache, const float *in, uint32_t pos, uint32_t dim, uint32_t batch);
/* scores[z][p][h] for p <= pos+z (other slots written as 0) */
void orc_mhsa(float *scores, const uint16_t *kcache, const float *q, uint32_t pos, uint32_t backlog, uint32_t heads,
              uint32_t rot, uint32_t batch);
void orc_softmax(float *scores, uint32_t pos, uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch);
void orc_kqv(float *out, const uint16_t *vcache, const float *attn, uint32_t backlog, uint32_t heads, uint32_t rot,
             uint32_t batch);
uint32_t orc_sample_greedy(const float *logits, uint32_t n);

/* ---- model level ---- */
typedef struct orc_model orc_model;
typedef struct orc_session orc_session;

typedef struct {
    uint32_t file_version, vocab, dim, multiple_of, heads, layers, rot, ftype, ff, n_tensors;
} orc_hparams;

orc_model *orc_model_open(const char *path);
void       orc_model_close(orc_model *m);
void       orc_model_hparams(const orc_model *m, orc_hparams *out);
/* tensor lookup by name with the reference's ".weight" fallback; returns 0 when found */
int orc_model_tensor(const orc_model *m, const char *name, uint32_t *ftype, uint64_t *offset, uint32_t *rows,
                     uint32_t *cols, uint64_t *size);
const void *orc_model_data(const orc_model *m, uint64_t offset);

orc_session *orc_session_new(const orc_model *m, uint32_t backlog);
void         orc_session_free(orc_session *s);
uint32_t     orc_session_pos(const orc_session *s);
void         orc_session_rewind(orc_session *s, uint32_t pos);
/* Evaluate n tokens as ONE batch at the session's current position (the reference's semantics for
 * batch > 1).  logits_last receives vocab floats of the last row; logits_all (optional) n*vocab. */
int orc_session_eval(orc_session *s, const uint32_t *tokens, uint32_t n, float *logits_last, float *logits_all);
/* raw fp16 cache rows [backlog][dim] of one layer (which: 0 = K, 1 = V) */
const uint16_t *orc_session_kv(const orc_session *s, uint32_t layer, int which);
/* restore n cache rows of one plane / set the position to continue from (snapshot restore) */
int orc_session_kv_load(orc_session *s, uint32_t layer, int which, const uint16_t *rows, uint32_t n);
int orc_session_set_pos(orc_session *s, uint32_t pos);
/* threads the checker's row loops run on */
int orc_num_threads(void);
/* per-layer intermediates of the LAST row of the last eval (trace); dim, ff or (which 5, the softmax weights
 * attn_result laid out [backlog][heads], llava_layer.cpp:60-61) backlog*heads floats */
const float *orc_session_trace(const orc_session *s, uint32_t layer, int which, uint32_t *count);

/* The same step in double precision: n tokens at positions pos0 .. pos0 + n - 1, logits of the last one.  Every sum,
 * product, exp, sin and cos in double, new cache rows rounded once to fp16; rows 0 .. pos0 - 1 of layer l are
 * kcache[l] / vcache[l] ([pos0][dim] fp16, may be null when pos0 is 0).  The yardstick two fp32 implementations are
 * measured against where their own difference is at the tolerance (pinned by an independent numpy forward pass). */
int orc_forward_f64(const orc_model *m, const uint32_t *tokens, uint32_t n, uint32_t pos0, const uint16_t *const *kcache,
                    const uint16_t *const *vcache, double *logits_last);

/* experiment knob of orc_forward_f64 (0 = off): quantise every GEMM input row per block of 32 to signed integers of `bits`
 * bits, as a kernel on the int8 matrix cores would; the logits' distance from the unquantised run prices such a kernel */
void orc_forward_f64_activation_bits(int bits);

#ifdef __cplusplus
}
#endif
#endif
