/*
 * llava_hip.h — C-ABI of the MI355X (gfx950) device layer that stands where the reference keeps its Vulkan
 * objects (llava_context / llava_device_memory / llava_buffer / llava_pipeline / llava_command_buffer).
 *
 * The reference's host classes that stay (ggml_file, llava_session, the server wrapper) call only the
 * functions below.  Everything is plain C: opaque handles, pointers and sizes.  Every function returns
 * LV_OK (0) or a negative lv_status; nothing throws and nothing aborts.  lv_last_error() gives the text of
 * the calling thread's last failure.
 *
 * Ownership: a handle belongs to whoever created it and is destroyed explicitly, children before parents
 * (sessions, then the model, then the context).  Host pointers are borrowed for the duration of the call.
 * All device work of a session runs on that session's own stream; a session must not be used from two
 * threads at once, different sessions of one model may be.  Weights are immutable after upload.
 *
 * Each declaration names the reference interface it replaces (paths relative to the reference tree).
 */
#ifndef LLAVA_HIP_H
#define LLAVA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    LV_OK = 0,
    LV_ERR_ARG = -1,      /* null pointer, bad shape, unsupported type */
    LV_ERR_HIP = -2,      /* a HIP runtime call failed; text in lv_last_error() */
    LV_ERR_OOM = -3,      /* device or host allocation failed */
    LV_ERR_STATE = -4,    /* call order violated (step already in flight, nothing to wait for, ...) */
    LV_ERR_RANGE = -5,    /* position / token id / backlog out of range */
    LV_ERR_MISSING = -6   /* a tensor the model needs is not in the table */
} lv_status;

/* GGML element types the layer understands (types.h:28-43 of the reference) */
enum { LV_F32 = 0, LV_F16 = 1, LV_Q4_0 = 2, LV_Q8_0 = 8 };

typedef struct lv_ctx lv_ctx;
typedef struct lv_model lv_model;
typedef struct lv_session lv_session;

const char *lv_last_error(void);

/* ---- device context: replaces instance/device/queue/pool bring-up, llava_context.cpp:230-282 ---------- */
int lv_ctx_create(int device, lv_ctx **out);
int lv_ctx_destroy(lv_ctx *ctx);
/* name, CU count, HBM bytes of the device (llava_context.cpp:240-251 prints the Vulkan equivalents) */
int lv_ctx_info(const lv_ctx *ctx, char *name, size_t name_cap, uint32_t *compute_units, uint64_t *hbm_bytes);

/* ---- model upload: replaces llava_layer::llava_layer + load_to_gpu (llava_layer.cpp:10-23,82-98),
 *      llava_buffer::load_from_disk (llava_buffer.cpp:179-325) and the per-session norm/output upload
 *      (llava_session.cpp:69-78).  One entry of the table per tensor of the GGJT file, exactly the fields of
 *      ggml_data_descriptor (ggml_file.h:29-41). ---------------------------------------------------------- */
typedef struct {
    const char *name;     /* e.g. "layers.0.attention.wq.weight" */
    uint32_t ftype;       /* LV_F32 / LV_Q4_0 / LV_Q8_0 */
    uint64_t offset;      /* byte offset of the payload from `base` */
    uint32_t rows, cols;  /* shape1, shape2: 2-D = (ne1, ne0); 1-D = (ne0, 1) */
    uint64_t size;        /* payload bytes */
} lv_tensor_desc;

typedef struct {
    uint32_t file_version;   /* 3 (fp16 block scales) or 1 (fp32 block scales, interleaved q4_0 nibbles) */
    uint32_t vocab, dim, heads, layers, rot, ff;
} lv_hparams;

/* Copies every tensor the decode path needs from the caller's mapping into an HBM weight arena (scales and
 * codes are split into two aligned streams on the way).  Synchronous: the mapping may go away afterwards
 * unless lv_step_begin is given token ids whose embedding rows live in it (see keep_host_embeddings). */
int lv_model_upload(lv_ctx *ctx, const void *base, uint64_t base_size, const lv_hparams *hp,
                    const lv_tensor_desc *table, uint32_t n_tensors, lv_model **out);
int lv_model_destroy(lv_model *model);
int lv_model_hparams(const lv_model *model, lv_hparams *out);
/* bytes of HBM the weight arena holds */
int lv_model_arena_bytes(const lv_model *model, uint64_t *bytes);

/* ---- session: replaces llava_session::recreate_buffers (llava_session.cpp:49-79), set_backlog_size
 *      (:303-327) and llava_layer_session_data::flush_buffers_on_gpu (llava_layer_session_data.cpp:52-163) */
int lv_session_create(lv_model *model, lv_session **out);
int lv_session_destroy(lv_session *s);
/* (re)size the fp16 K/V caches to `backlog` rows per layer (any value >= 1; the reference uses powers of two
 * 128..2048): the first min(old,new) rows are kept, the rest zero-filled.  Waits for the stream. */
int lv_session_reserve(lv_session *s, uint32_t backlog);
int lv_session_backlog(const lv_session *s, uint32_t *backlog);

/* ---- one step: replaces the body of llava_session::start_next_token_prediction (llava_session.cpp:197-229),
 *      llava_command_buffer::record_execution / run (llava_command_buffer.cpp:29-55) and the whole shader chain
 *      of llava_layer::execute (llava_layer.cpp:39-75).
 *      Asynchronous.  Evaluates n tokens whose cache rows are pos .. pos+n-1 (pos = tokens already cached).
 *      Row z attends to cache rows 0 .. pos+z, like the batched shaders.  n == 1 replays a captured hipGraph. */
int lv_step_begin(lv_session *s, const uint32_t *token_ids, uint32_t n, uint32_t pos);
/* replaces llava_command_buffer::wait_idle (llava_command_buffer.cpp:25-27): the only sync point */
int lv_step_wait(lv_session *s);
/* replaces output_probs->map in get_last_predicted_token (llava_session.cpp:129-135): logits of the LAST row
 * of the last step, `vocab` floats.  Implies lv_step_wait. */
int lv_logits_read(lv_session *s, float *dst);
/* The reference computes the logits of EVERY row of a step (output_probs is batch x vocab, llava_session.cpp:49-79; the
 * head runs over all rows, llava_command_buffer.cpp:38-39) and its interface reads the last (llava_session.cpp:131-135).
 * With this switch on, a step keeps all of them on the device and lv_logits_read_rows returns rows row0 .. row0 + n_rows - 1
 * of the last step (row z = the token at position pos + z), `vocab` floats each; implies lv_step_wait.  Off by default:
 * a 512-token prompt then multiplies one row by the output matrix instead of 512. */
int lv_session_set_all_logits(lv_session *s, int enable);
int lv_logits_read_rows(lv_session *s, uint32_t row0, uint32_t n_rows, float *dst);
/* index of the first strict maximum of those logits, computed on the device (the greedy rule of
 * llava_session.cpp:144-152).  Implies lv_step_wait. */
int lv_argmax(lv_session *s, uint32_t *token);
/* Enables/disables hipGraph replay for n == 1 steps (on by default); off = plain stream launches. */
int lv_session_use_graph(lv_session *s, int enable);
/* How n == 1 steps are executed.  The reference has one way (replay the recorded command buffers,
 * llava_command_buffer.cpp:47-55); here there are three, all computing the same step:
 *   LV_PATH_KERNELS     one launch per operator on the session's stream
 *   LV_PATH_GRAPH       the same launches captured once into a hipGraph and replayed
 *   LV_PATH_PERSISTENT  one persistent kernel for the whole token (LLaMA-7B and -13B layer shapes, q4_0 or q8_0, on a
 *                       256-CU device)
 *   LV_PATH_AUTO        persistent when the model has that form, else graph (or kernels if graphs are off)
 * A session stops using the persistent kernel, and lv_session_path reports the graph path (kernels if graphs are off)
 * from then on, when its 256 workgroups cannot all be resident on the device (the step goes on in the other path and succeeds) or when
 * two steps in a row end with an expired hand-over wait (both report LV_ERR_HIP; the step issued again then succeeds).
 * lv_session_set_path(LV_PATH_PERSISTENT) gives the kernel another try. */
enum { LV_PATH_AUTO = 0, LV_PATH_KERNELS = 1, LV_PATH_GRAPH = 2, LV_PATH_PERSISTENT = 3 };
int lv_session_set_path(lv_session *s, int path);
int lv_session_path(const lv_session *s, int *path);
/* Workgroups of the persistent kernel wait for each other's results by polling, a bounded number of times; a wait
 * that runs out makes the kernel finish anyway and lv_step_wait return LV_ERR_HIP (the reference's waitForFences
 * timeout, llava_command_buffer.cpp:25-27, is the nearest counterpart).  polls = 0 restores the default bound; tests of
 * that failure path set 1.  The step can simply be issued again afterwards; after two such steps in a row it runs in
 * the graph path (see lv_session_set_path). */
int lv_session_set_wait_limit(lv_session *s, uint32_t polls);
/* The persistent kernel hands a head's query, key and value rows and its partial sums over inside one XCD (through that
 * XCD's L2 instead of memory) whenever a launch has placed the workgroups that share heads on one XCD; it looks at every
 * launch and falls back to device scope by itself.  enable = 0 keeps every launch at device scope (for comparison and
 * diagnosis; results are bit-identical either way).  lv_session_xcd_handover tells what the session's last persistent
 * step did (0 before one).  No counterpart in the reference, which has one queue and no such choice. */
int lv_session_set_xcd_handover(lv_session *s, int enable);
int lv_session_xcd_handover(lv_session *s, int *used);

/* ---- cache dump / restore: replaces llava_layer_session_data::dump_kv_cache / restore_kv_cache
 *      (llava_layer_session_data.cpp:165-181).  which: 0 = K, 1 = V.  n_tokens rows of `dim` fp16 values. */
int lv_kv_read(lv_session *s, uint32_t layer, int which, uint32_t n_tokens, void *dst);
int lv_kv_write(lv_session *s, uint32_t layer, int which, uint32_t n_tokens, const void *src);

/* ---- record mode: replaces the per-layer trace buffers of llava_layer_session_data.cpp:79-86 and their
 *      routing in llava_layer.cpp:43-51.  When enabled, every step keeps, per layer and for every row of the step (the
 *      reference's buffers are batch_size rows long, llava_layer_session_data.cpp:80-85), the LV_TRACE_* below; the
 *      next step replaces them.  Memory: layers x rows x (5 x max(dim, ff) + backlog x heads) floats, grown to the
 *      longest step recorded so far. */
enum {
    LV_TRACE_NORM_IN = 0,        /* normalized_input_logit  [dim] */
    LV_TRACE_POST_ATTN = 1,      /* post_attn_logit         [dim] */
    LV_TRACE_POST_ATTN_NORM = 2, /* post_attn_norm_logit    [dim] */
    LV_TRACE_FF = 3,             /* ff_result               [ff]  */
    LV_TRACE_OUT = 4,            /* output_logit            [dim] */
    LV_TRACE_ATTN = 5,           /* attn_result             [backlog][heads]: softmax weights, 0 behind the row's position
                                    (mhsa.comp + softmax.comp; the reference's [BACKLOG][HEAD_COUNT] layout) */
    LV_TRACE_COUNT = 6
};
int lv_trace_enable(lv_session *s, int enable);
/* rows of the last recorded step (0 before the first) */
int lv_trace_rows(lv_session *s, uint32_t *rows);
/* rows [row0, row0 + n_rows) of one buffer of the last recorded step to the host, row after row with nothing between
 * them: the memory layout of the reference's buffer (z_id * dim, z_id * BACKLOG * HEAD_COUNT: mhsa.comp:58) */
int lv_trace_read_rows(lv_session *s, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, float *dst);
/* the last row of the last recorded step (count = the floats of one row) */
int lv_trace_read(lv_session *s, uint32_t layer, int which, float *dst, uint32_t count);

/* ---- device memory helpers for callers of the lv_kernel_* entry points (tests, microbenchmarks) -------- */
int lv_dev_alloc(lv_ctx *ctx, uint64_t bytes, void **dptr);
int lv_dev_free(lv_ctx *ctx, void *dptr);
int lv_dev_upload(lv_ctx *ctx, void *dptr, const void *src, uint64_t bytes);
int lv_dev_download(lv_ctx *ctx, void *dst, const void *dptr, uint64_t bytes);
int lv_dev_zero(lv_ctx *ctx, void *dptr, uint64_t bytes);
/* device-to-device copy on the context's stream (asynchronous); size and pointers multiples of 16 */
int lv_dev_copy(lv_ctx *ctx, void *dst, const void *src, uint64_t bytes);
/* read-only pass over device memory on the context's stream (asynchronous), the result discarded: with lv_ctx_timer_* it
 * gives the read bandwidth this device reaches, the denominator a weight-streaming kernel is also measured against
 * (no counterpart in the reference: a measuring aid like the timers); size and pointer multiples of 16 */
int lv_dev_read(lv_ctx *ctx, const void *src, uint64_t bytes);
int lv_ctx_sync(lv_ctx *ctx);

/* ---- GPU time between two points of a stream, by HIP events recorded on that very stream (the reference has
 *      no timers at all; benchmarks need them).  stop waits for the stream and returns milliseconds. ------- */
int lv_ctx_timer_start(lv_ctx *ctx);
int lv_ctx_timer_stop(lv_ctx *ctx, float *ms);
int lv_session_timer_start(lv_session *s);
int lv_session_timer_stop(lv_session *s, float *ms);

/* A quantised matrix in the device layout.  Built from GGML blocks by lv_matrix_upload; owns its memory. */
typedef struct lv_matrix lv_matrix;
/* replaces llava_buffer::load_from_disk for one tensor (llava_buffer.cpp:179-325).  file_version 3: 18 / 34-byte blocks
 * with an fp16 scale; file_version 1 (llava_buffer.cpp:193-224, ggml_file.cpp:171-183): 20 / 36-byte blocks with an fp32
 * scale, q4_0 byte j holding elements 2j and 2j+1; the device keeps an fp32 scale plane for such a matrix. */
int lv_matrix_upload(lv_ctx *ctx, const void *ggml_blocks, uint32_t ftype, uint32_t file_version, uint32_t rows,
                     uint32_t cols, lv_matrix **out);
int lv_matrix_destroy(lv_matrix *m);
/* bytes the device layout occupies (equals the GGML payload size: 18 / 34 bytes per 32 weights, 20 / 36 for file version 1) */
int lv_matrix_bytes(const lv_matrix *m, uint64_t *bytes);

/* ---- single kernels on the context's stream; all pointers are device pointers.  Asynchronous: follow with
 *      lv_ctx_sync.  `batch` rows are independent (the shaders' gl_GlobalInvocationID.z). ------------------- */

/* dequantise rows [row0, row0+n_rows) of m to fp32: the arithmetic of llava_buffer::write_f32
 * (llava_buffer.cpp:339-401), bit-exact */
int lv_kernel_dequant(lv_ctx *ctx, const lv_matrix *m, uint32_t row0, uint32_t n_rows, float *dst);
/* matmul_dim* / matmul_ff* (matmul.glsl:41-74, matmul_q8.glsl:41-72); accumulate != 0 = matmul_add_* */
int lv_kernel_gemv(lv_ctx *ctx, float *out, const lv_matrix *w, const float *x, uint32_t batch, int accumulate);
/* the same product for many rows at once on the matrix cores: the *_batch variants of the shaders the reference
 * switches to when several tokens are pending (llava_session.cpp:243-255, llava_pipeline.cpp batch_enabled).
 * out[batch][rows] (+)= x[batch][cols] * W^T.  The first call on a matrix makes its prompt copy (2 bytes a weight, kept
 * until lv_matrix_destroy); the activation workspace belongs to the context and only grows.  Neither is allocated again
 * by later calls of the same size, which are asynchronous like the other kernels. */
int lv_kernel_gemm(lv_ctx *ctx, float *out, const lv_matrix *w, const float *x, uint32_t batch, int accumulate);
/* matmul_silu_ff* (matmul_silu_ff.comp:49-97): out = (W3 x) * silu(W1 x) */
int lv_kernel_gemv_silu(lv_ctx *ctx, float *out, const lv_matrix *w3, const lv_matrix *w1, const float *x,
                        uint32_t batch);
/* normalize (normalize.comp:34-64): out = x * w * rsqrt(mean((x - mean(x))^2)), no epsilon */
int lv_kernel_normalize(lv_ctx *ctx, float *out, const float *x, const float *w, uint32_t dim, uint32_t batch);
/* copy_to_cache (copy_to_cache.comp:29-37): cache[(pos+z)*dim + i] = fp16(in[z*dim + i]) */
int lv_kernel_kv_append(lv_ctx *ctx, void *cache, const float *in, uint32_t pos, uint32_t dim, uint32_t batch,
                        uint32_t backlog);
/* mhsa + softmax + kqv_matching fused (mhsa.comp:32-60, softmax.comp:26-44, kqv_matching.comp:27-42):
 * out[z][dim] = sum_{p <= pos+z} softmax_p( Q_z . Rot(-(pos+z-p) theta) K_p / sqrt(rot) ) V_p  per head.
 * Up to 15 rows go through the one-query kernel of the decode path, 16 and more through the kernels of a prompt batch
 * (matrix cores on exact 16-bit pieces of the fp32 operands); the two agree to about 1e-6 of the largest output. */
int lv_kernel_attention(lv_ctx *ctx, float *out, const void *kcache, const void *vcache, const float *q,
                        uint32_t pos, uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch);

/* lv_kernel_attention for callers that cannot allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same result (the one-query
 * kernel at every batch size); the rotation
 * table, the partial sums and the split counters live in a fixed 2 MiB work area that every device holds from library
 * load to process end, so the call allocates nothing and frees nothing.  Limits (LV_ERR_RANGE beyond them):
 * backlog * rot / 2 <= 131072, batch * heads * ceil(backlog / 64) * (rot + 1) <= 262144, batch * heads <= 256.
 * Every call rewrites the rotation table for its backlog and head size (a small kernel in front of the attention: up to
 * 1 MiB written) and clears the split counters, so nothing is carried from call to call.
 * All calls on one device share the work area: calls that overlap on one device (different contexts, different threads)
 * race; calls on one context are ordered by its stream. */
int lv_kernel_attention_static(lv_ctx *ctx, float *out, const void *kcache, const void *vcache, const float *q,
                               uint32_t pos, uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch);

#ifdef __cplusplus
}
#endif
#endif /* LLAVA_HIP_H */
