// lv_api.hip — implementation of the C-ABI declared in include/llava_hip.h for gfx950.
//
// What lives here: the HBM weight arena and its upload path, per-session K/V cache + activation buffers on
// one stream, the decode step as a chain of hand-written kernels (lv_kernels.h) captured into a hipGraph,
// and thin single-kernel entry points.  No Vulkan-style objects survive: a "buffer" is a pointer into an
// arena, a "pipeline" is a template instantiation, the "command buffer" is the captured graph.
#include "../../include/llava_hip.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "lv_kernels.h"
#include "lv_mega.h"
#include "lv_gemm.h"
#include "lv_gemv_wide.h"
#include "lv_attn_batch.h"

using namespace lv;

// -----------------------------------------------------------------------------------------------------------
// errors
// -----------------------------------------------------------------------------------------------------------
static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                                         \
    do {                                                                                                      \
        hipError_t e_ = (expr);                                                                               \
        if (e_ != hipSuccess) return fail(LV_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                                          __FILE__, __LINE__);                                                \
    } while (0)

#define LV_TRY(expr)              \
    do {                          \
        int rc_ = (expr);         \
        if (rc_ != LV_OK) return rc_; \
    } while (0)

extern "C" const char *lv_last_error(void) { return g_err; }

// -----------------------------------------------------------------------------------------------------------
// objects
// -----------------------------------------------------------------------------------------------------------
struct lv_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
    // scratch for the stand-alone attention entry point
    float2 *trig = nullptr;
    uint32_t trig_rows = 0, trig_rot = 0;
    float *attn_part = nullptr;
    uint32_t *attn_counters = nullptr;
    size_t attn_part_floats = 0, attn_counter_words = 0;
    // and for its batched form (batch >= kPrefillMin): absolute-position table and operand planes
    float2 *trig_abs = nullptr;
    uint32_t trig_abs_rows = 0, trig_abs_rot = 0;
    uint16_t *attn_planes = nullptr;
    size_t attn_plane_halfs = 0;
    // workspace of the stand-alone GEMM entry point (activation halves, row scales, K-slice partials); grows, never shrinks
    uint16_t *gemm_ws = nullptr;
    size_t gemm_ws_bytes = 0;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    uint32_t *read_sink = nullptr;       // where lv_dev_read's kernel could leave a word
    struct AttnScratch *scratch = nullptr;   // this device's copy of the file-scope scratch array (lv_kernel_attention_static)
    // Persistent decode kernels of different sessions (one per thread, llava_context.h:47-49 has the same pools and
    // mutexes for the same reason) must not overlap on the device: each occupies every CU and its workgroups wait
    // for each other.  A launch on another session's stream first waits for the event the last launch recorded.
    std::mutex mega_mutex;
    hipEvent_t mega_done = nullptr;
    const void *mega_last = nullptr;      // session whose launch mega_done belongs to
    int mega_fits[8] = {-1, -1, -1, -1, -1, -1, -1, -1};   // per shape class of the persistent kernel: can all its workgroups be resident at once (-1 = not asked yet)
};

struct lv_matrix {
    lv_ctx *ctx = nullptr;
    void *owned = nullptr;  // allocation to free, or null when the matrix lives in a model arena
    MatView view{};
    uint32_t ftype = 0;
    uint64_t bytes = 0;
    mutable const uint16_t *h16 = nullptr;   // prompt copy (lv_gemm.h): codes as fp16 integers and fp32 scales in tile order; null until a batch needs it
    mutable uint16_t *h16_owned = nullptr;   // that copy when lv_kernel_gemm made it for a matrix outside a model; freed with the matrix
};

// Uncached device memory (hipDeviceMallocUncached) for the persistent kernel's device-wide hand-over vectors.  Such memory
// is never given back to the runtime once a kernel has read it (allocations made after such a free have been seen to hold
// wrong values); a session that ends leaves its buffers here for the next one of the same size.
struct UncachedBlock { int device; size_t bytes; void *ptr; };
static std::mutex g_uncached_mutex;
static std::vector<UncachedBlock> g_uncached_free;

static int uncached_take(int device, void **out, size_t bytes, bool *pooled)
{
    *pooled = true;
    {
        std::lock_guard<std::mutex> lock(g_uncached_mutex);
        for (size_t i = 0; i < g_uncached_free.size(); i++)
            if (g_uncached_free[i].device == device && g_uncached_free[i].bytes == bytes) {
                *out = g_uncached_free[i].ptr;
                g_uncached_free.erase(g_uncached_free.begin() + (long)i);
                return LV_OK;
            }
    }
    hipError_t e = hipExtMallocWithFlags(out, bytes, hipDeviceMallocUncached);
    if (e != hipSuccess) {
        // a runtime without that kind of memory: ordinary memory does as well, only slower (the hand-overs are device scope
        // either way); such a block is freed like any other
        (void)hipGetLastError();
        *pooled = false;
        e = hipMalloc(out, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "hand-over buffer of %llu bytes: %s", (unsigned long long)bytes, hipGetErrorString(e));
    }
    return LV_OK;
}

static void uncached_give(int device, void *ptr, size_t bytes, bool pooled)
{
    if (!ptr) return;
    if (!pooled) {
        (void)hipFree(ptr);
        return;
    }
    std::lock_guard<std::mutex> lock(g_uncached_mutex);
    g_uncached_free.push_back({device, bytes, ptr});
}

struct LayerWeights {
    lv_matrix wq, wk, wv, wo, w1, w2, w3;
    const float *attn_norm = nullptr, *ffn_norm = nullptr;
    const uint16_t *gate_up16 = nullptr;   // pair copy of w3 and w1 (in place of their own prompt copies) where they can share one
};

struct lv_model {
    lv_ctx *ctx = nullptr;
    lv_hparams hp{};
    uint8_t *arena = nullptr;
    uint64_t arena_bytes = 0;
    std::vector<LayerWeights> layers;
    const float *norm = nullptr;
    lv_matrix output;
    uint32_t tok_ftype = LV_F32;
    const float *tok_f32 = nullptr;
    lv_matrix tok_quant;
    // persistent-kernel form of the weights (null when the model's shape has no compiled MegaShape)
    int mega_kind = 0;              // 0 none, else a compiled shape class of the persistent kernel (mega_dispatch)
    uint8_t *mega_stream = nullptr;
    float *mega_norms = nullptr;    // [layers][2][D] + final norm [D]
    float *tok_f32_own = nullptr;   // fp32 copy of a quantised embedding table (the persistent kernel reads rows as fp32)
    // prompt copy of the layer matrices (lv_gemm.h), made when the first batch is evaluated; sessions of several threads share it
    std::mutex prompt_mutex;
    int prompt_state = 0;           // 0 not made yet, 1 ready, -1 could not be made (batches then go token by token)
    uint16_t *prompt_arena = nullptr;
    int output_state = 0;           // the same for the prompt copy of the output matrix, which only steps that keep every row's logits need
    uint16_t *output_copy = nullptr;
};

// Shape classes the persistent kernel is compiled for: LLaMA-7B and LLaMA-13B layer shapes, q4_0 and q8_0.
// Eight wavefronts per workgroup (two per SIMD leave each wave 256 registers, which buys a queue 8 q4_0 tiles or 4 q8_0 tiles
// deep; twelve waves with the shallow queue the register file then allows lost 6-13 %).  The 13B classes ran on seven waves
// while a wave was tied to one of three column slabs, the third half empty; with the half slab's tiles carrying two rows
// and the waves dealt 3 + 3 + 2 (MegaShapeBase) all eight work in the D-wide phases: 13B q4_0 544 -> 592-607 tok/s, 13B q8_0
// 357-370 -> 379-392.
using Mega7Bq4 = MegaShape<4096, 11008, 32, 8, 4, 8>;
using Mega7Bq8 = MegaShape<4096, 11008, 32, 8, 8, 4>;
using Mega13Bq4 = MegaShape<5120, 13824, 40, 8, 4, 8>;
using Mega13Bq8 = MegaShape<5120, 13824, 40, 8, 8, 4>;
// the same for version-1 files (fp32 block scales; the reference loads q4_0 of that version only, llava_buffer.cpp:66-71)
using Mega7Bq4v1 = MegaShapeV1<4096, 11008, 32, 8, 4, 8>;
using Mega13Bq4v1 = MegaShapeV1<5120, 13824, 40, 8, 4, 8>;
constexpr int kMegaKinds = 6;

template <class Fn>
static int mega_dispatch(int kind, Fn &&fn)
{
    switch (kind) {
    case 1: return fn(Mega7Bq4{});
    case 2: return fn(Mega7Bq8{});
    case 3: return fn(Mega13Bq4{});
    case 4: return fn(Mega13Bq8{});
    case 5: return fn(Mega7Bq4v1{});
    case 6: return fn(Mega13Bq4v1{});
    default: return fail(LV_ERR_STATE, "no persistent kernel for this model");
    }
}

constexpr uint32_t kAttnChunk = kAttnChunkRows;   // cache positions per attention workgroup
constexpr uint32_t kMaxStepTokens = 4096;

struct lv_session {
    lv_model *model = nullptr;
    hipStream_t stream = nullptr;
    uint32_t backlog = 0;
    uint16_t *kv = nullptr;  // [layers][2][backlog][dim]
    float2 *trig = nullptr;  // [backlog][rot/2]: cos/sin of delta * theta_i as the shader evaluates it
    float2 *trig_abs = nullptr;  // [backlog][rot/2]: cos/sin of p * theta_i (batched attention)
    // activations (batch 1)
    float *x = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *vo = nullptr, *ff = nullptr,
          *logits = nullptr;
    float *attn_part = nullptr;
    uint32_t *attn_counters = nullptr;
    uint32_t *cfg = nullptr;       // device: [0] = pos, [1..] = token ids of the step
    uint32_t *cfg_host = nullptr;  // pinned staging of the same
    uint32_t *argmax_dev = nullptr;
    uint32_t *argmax_host = nullptr;  // pinned
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    bool use_graph = true;
    int path = LV_PATH_AUTO;
    // workspace of the batched prompt path, allocated at first use: activations for pf_cap tokens
    uint32_t pf_cap = 0;
    float *pf_x = nullptr, *pf_xn = nullptr, *pf_q = nullptr, *pf_k = nullptr, *pf_v = nullptr, *pf_vo = nullptr, *pf_g1 = nullptr, *pf_g2 = nullptr;
    uint16_t *pf_xh = nullptr, *pf_xl = nullptr;
    uint16_t *pf_fh = nullptr, *pf_fl = nullptr;   // the feed-forward's inner activations (their producer still reads pf_xh / pf_xl)
    float *pf_xs = nullptr;   // per token: the power of two the halves written by prefill_norm_kernel are scaled down by
    // operand planes of the batched attention (one layer's worth, rewritten per layer): four of attn_plane_halfs() each
    uint16_t *pf_planes = nullptr;
    size_t pf_plane_halfs = 0;
    float *xchg[2] = {nullptr, nullptr};  // hand-over buffer sets of the persistent kernel: uncached memory (uncached_take / uncached_give) ...
    size_t xchg_bytes = 0;
    bool xchg_pooled[2] = {true, true};   // false: the runtime had no uncached memory and the set lies in ordinary memory
    float *xl[2] = {nullptr, nullptr};    // ... and the part of them that stays inside an XCD, ordinary memory
    uint32_t xchg_turn = 0;
    uint32_t *status_host = nullptr;      // pinned, written by the persistent kernel: [0] a poll expired, [kStatusToken] greedy pick
    uint32_t wait_limit = 0;              // polls per hand-over of the persistent kernel; 0 = default
    bool xcd_handover = true;             // the persistent kernel may keep a head's hand-overs inside its XCD (lv_session_set_xcd_handover)
    bool pick_in_status = false;          // the last step ran the persistent kernel, whose greedy pick is in status_host
    bool mega_step = false;               // the step in flight ran the persistent kernel
    int mega_failures = 0;                // steps of the persistent kernel in a row that ended with an expired wait
    bool mega_off = false;                // the persistent kernel is no longer used by this session (refused launch, or two such steps)
    bool in_flight = false;
    bool have_logits = false;
    // logits of EVERY row of a step (the reference's output_probs holds batch x vocab, llava_session.cpp:49-79), kept on request
    bool all_logits = false;
    float *logits_all = nullptr;          // [logits_cap][vocab]
    uint32_t logits_cap = 0, logits_rows = 0;
    bool trace = false;
    // record mode keeps every row of a step, as the reference's batch-sized buffers do (llava_layer_session_data.cpp:79-86)
    float *trace_buf = nullptr;  // [layers][LV_TRACE_ATTN][trace_cap][max(dim, ff)]: the five vector buffers
    float *trace_attn = nullptr; // [layers][trace_cap][backlog][heads]: LV_TRACE_ATTN; follows the backlog
    uint32_t trace_cap = 0;      // rows the two buffers have room for
    uint32_t trace_n = 0;        // rows the last recorded step wrote
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
};

static uint16_t *kv_ptr(const lv_session *s, uint32_t layer, int which)
{
    const size_t plane = (size_t)s->backlog * s->model->hp.dim;
    return s->kv + ((size_t)layer * 2 + (which ? 1 : 0)) * plane;
}

// -----------------------------------------------------------------------------------------------------------
// Device memory that exists without any allocation call: the work area of lv_kernel_attention_static, for callers that
// may not allocate.  Every device the library runs on holds its own copy from the moment the code object is loaded until
// the process ends.  Host code never uses the array's name as an address: lv_ctx_create asks the runtime for this
// device's copy once (hipGetSymbolAddress) and keeps the pointer in the context.
// -----------------------------------------------------------------------------------------------------------
constexpr uint32_t kStaticTrigPairs = 131072;   // rotation table: backlog * rot / 2 (cos, sin) pairs (2048 rows of a 128-wide head)
constexpr uint32_t kStaticPartFloats = 262144;  // partial sums: batch * heads * ceil(backlog / 64) * (rot + 1)
constexpr uint32_t kStaticCounters = 256;       // batch * heads
struct AttnScratch {
    float2 trig[kStaticTrigPairs];
    float part[kStaticPartFloats];
    uint32_t counters[kStaticCounters];
};
static __device__ __align__(256) unsigned char scratch[sizeof(AttnScratch)];   // 2 MiB + 1 KiB

// -----------------------------------------------------------------------------------------------------------
// context
// -----------------------------------------------------------------------------------------------------------
extern "C" int lv_ctx_create(int device, lv_ctx **out)
{
    if (!out) return fail(LV_ERR_ARG, "lv_ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(LV_ERR_ARG, "lv_ctx_create: device %d of %d", device, count);
    HIP_TRY(hipSetDevice(device));
    lv_ctx *c = new (std::nothrow) lv_ctx;
    if (!c) return fail(LV_ERR_OOM, "lv_ctx_create: host allocation");
    c->device = device;
    hipError_t e = hipGetDeviceProperties(&c->props, device);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    // the address of the scratch array on THIS device (the current one); each device has its own copy at its own address
    if (e == hipSuccess) e = hipGetSymbolAddress(reinterpret_cast<void **>(&c->scratch), HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return fail(LV_ERR_HIP, "lv_ctx_create: %s", hipGetErrorString(e));
    }
    *out = c;
    return LV_OK;
}

extern "C" int lv_ctx_destroy(lv_ctx *c)
{
    if (!c) return LV_OK;
    (void)hipSetDevice(c->device);
    (void)hipStreamSynchronize(c->stream);
    (void)hipFree(c->trig);
    (void)hipFree(c->attn_part);
    (void)hipFree(c->attn_counters);
    (void)hipFree(c->trig_abs);
    (void)hipFree(c->attn_planes);
    (void)hipFree(c->gemm_ws);
    (void)hipFree(c->read_sink);
    if (c->ev_start) (void)hipEventDestroy(c->ev_start);
    if (c->ev_stop) (void)hipEventDestroy(c->ev_stop);
    if (c->mega_done) (void)hipEventDestroy(c->mega_done);
    (void)hipStreamDestroy(c->stream);
    delete c;
    return LV_OK;
}

extern "C" int lv_ctx_info(const lv_ctx *c, char *name, size_t cap, uint32_t *cus, uint64_t *hbm)
{
    if (!c) return fail(LV_ERR_ARG, "lv_ctx_info: ctx is null");
    if (name && cap) {
        if (c->props.name[0]) snprintf(name, cap, "%s (%s)", c->props.name, c->props.gcnArchName);
        else snprintf(name, cap, "%s", c->props.gcnArchName);  // some driver set-ups report no marketing name
    }
    if (cus) *cus = (uint32_t)c->props.multiProcessorCount;
    if (hbm) *hbm = (uint64_t)c->props.totalGlobalMem;
    return LV_OK;
}

extern "C" int lv_ctx_sync(lv_ctx *c)
{
    if (!c) return fail(LV_ERR_ARG, "lv_ctx_sync: ctx is null");
    HIP_TRY(hipStreamSynchronize(c->stream));
    return LV_OK;
}

// ---- stream timers ---------------------------------------------------------------------------------------
static int timer_start(hipEvent_t *a, hipEvent_t *b, hipStream_t st)
{
    if (!*a) HIP_TRY(hipEventCreate(a));
    if (!*b) HIP_TRY(hipEventCreate(b));
    HIP_TRY(hipEventRecord(*a, st));
    return LV_OK;
}

static int timer_stop(hipEvent_t a, hipEvent_t b, hipStream_t st, float *ms)
{
    if (!a || !b) return fail(LV_ERR_STATE, "timer stop without start");
    HIP_TRY(hipEventRecord(b, st));
    HIP_TRY(hipEventSynchronize(b));
    HIP_TRY(hipEventElapsedTime(ms, a, b));
    return LV_OK;
}

extern "C" int lv_ctx_timer_start(lv_ctx *c)
{
    if (!c) return fail(LV_ERR_ARG, "lv_ctx_timer_start: ctx is null");
    return timer_start(&c->ev_start, &c->ev_stop, c->stream);
}

extern "C" int lv_ctx_timer_stop(lv_ctx *c, float *ms)
{
    if (!c || !ms) return fail(LV_ERR_ARG, "lv_ctx_timer_stop: null argument");
    return timer_stop(c->ev_start, c->ev_stop, c->stream, ms);
}

extern "C" int lv_dev_alloc(lv_ctx *c, uint64_t bytes, void **dptr)
{
    if (!c || !dptr) return fail(LV_ERR_ARG, "lv_dev_alloc: null argument");
    *dptr = nullptr;
    if (bytes == 0) return LV_OK;
    hipError_t e = hipMalloc(dptr, bytes);
    if (e == hipErrorOutOfMemory) return fail(LV_ERR_OOM, "lv_dev_alloc: %llu bytes", (unsigned long long)bytes);
    HIP_TRY(e);
    return LV_OK;
}

extern "C" int lv_dev_free(lv_ctx *c, void *dptr)
{
    if (!c) return fail(LV_ERR_ARG, "lv_dev_free: ctx is null");
    if (dptr) HIP_TRY(hipFree(dptr));
    return LV_OK;
}

extern "C" int lv_dev_upload(lv_ctx *c, void *dptr, const void *src, uint64_t bytes)
{
    if (!c || (bytes && (!dptr || !src))) return fail(LV_ERR_ARG, "lv_dev_upload: null argument");
    if (bytes == 0) return LV_OK;
    HIP_TRY(hipMemcpyAsync(dptr, src, bytes, hipMemcpyHostToDevice, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return LV_OK;
}

extern "C" int lv_dev_download(lv_ctx *c, void *dst, const void *dptr, uint64_t bytes)
{
    if (!c || (bytes && (!dptr || !dst))) return fail(LV_ERR_ARG, "lv_dev_download: null argument");
    if (bytes == 0) return LV_OK;
    HIP_TRY(hipMemcpyAsync(dst, dptr, bytes, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return LV_OK;
}

// zero fill with a kernel (usable inside graph capture, unlike a memset node)
__global__ void fill_zero_kernel(uint32_t *p, uint64_t words)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (uint64_t)gridDim.x * blockDim.x)
        p[i] = 0u;
}

static int zero_async(void *p, uint64_t bytes, hipStream_t st)
{
    if (bytes == 0) return LV_OK;
    if (bytes % 4) return fail(LV_ERR_ARG, "zero fill: size not a multiple of 4");
    const uint64_t words = bytes / 4;
    uint64_t blocks = (words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_zero_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(static_cast<uint32_t *>(p), words);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

extern "C" int lv_dev_zero(lv_ctx *c, void *dptr, uint64_t bytes)
{
    if (!c || (bytes && !dptr)) return fail(LV_ERR_ARG, "lv_dev_zero: null argument");
    return zero_async(dptr, bytes, c->stream);
}

// plain device-to-device copy (16 bytes per thread per pass): the yardstick for achievable HBM bandwidth and for
// calibrating hardware traffic counters
__global__ void copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, uint64_t n16)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

extern "C" int lv_dev_copy(lv_ctx *c, void *dst, const void *src, uint64_t bytes)
{
    if (!c || (bytes && (!dst || !src))) return fail(LV_ERR_ARG, "lv_dev_copy: null argument");
    if (bytes % 16 || ((uintptr_t)dst | (uintptr_t)src) % 16) return fail(LV_ERR_ARG, "lv_dev_copy: size and pointers must be multiples of 16");
    if (bytes == 0) return LV_OK;
    copy_kernel<<<dim3(256 * 16), dim3(256), 0, c->stream>>>(static_cast<uint4 *>(dst), static_cast<const uint4 *>(src), bytes / 16);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// Read-only stream: every workgroup walks its own contiguous share of the buffer, 16 bytes a thread and load, eight loads in
// flight, non-temporal like the decode kernel's weight tiles; the XOR of everything read leaves for `sink` so that no load can
// be dropped.  What a kernel that only has to READ memory can reach on this device: the second denominator next to the 8 TB/s
// on the datasheet.
__global__ __launch_bounds__(256) void read_stream_kernel(const uint4 *__restrict__ src, uint64_t n16, uint32_t *__restrict__ sink)
{
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    const uint64_t per = (n16 + gridDim.x - 1) / gridDim.x, lo = (uint64_t)blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
    const u4v *p = reinterpret_cast<const u4v *>(src);
    u4v acc = {0u, 0u, 0u, 0u};
    uint64_t i = lo + threadIdx.x;
    for (; i + 7 * 256 < hi; i += 8 * 256) {
        u4v v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = __builtin_nontemporal_load(p + i + j * 256);
#pragma unroll
        for (int j = 0; j < 8; j++) acc ^= v[j];
    }
    for (; i < hi; i += 256) acc ^= __builtin_nontemporal_load(p + i);
    const uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (x == 0x9e3779b9u) sink[blockIdx.x & 255] = x;      // practically never taken; keeps the loads alive
}

extern "C" int lv_dev_read(lv_ctx *c, const void *src, uint64_t bytes)
{
    if (!c || (bytes && !src)) return fail(LV_ERR_ARG, "lv_dev_read: null argument");
    if (bytes % 16 || (uintptr_t)src % 16) return fail(LV_ERR_ARG, "lv_dev_read: size and pointer must be multiples of 16");
    if (bytes == 0) return LV_OK;
    if (!c->read_sink) HIP_TRY(hipMalloc(reinterpret_cast<void **>(&c->read_sink), 256 * 4));
    read_stream_kernel<<<dim3(256 * 8), dim3(256), 0, c->stream>>>(static_cast<const uint4 *>(src), bytes / 16, c->read_sink);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// matrices
// -----------------------------------------------------------------------------------------------------------
// bytes of n elements in the file (ggml_file.cpp:162-186): version-1 files carry fp32 block scales, 2 bytes more a block
static uint64_t ggml_bytes(uint32_t ftype, uint64_t n, uint32_t file_version)
{
    const uint64_t wide = file_version == 1 ? 2 : 0;
    switch (ftype) {
    case LV_F32: return n * 4;
    case LV_F16: return n * 2;
    case LV_Q4_0: return n / 32 * (18 + wide);
    case LV_Q8_0: return n / 32 * (34 + wide);
    default: return 0;
    }
}

// device bytes of the split layout: codes first (16-byte aligned), scales after (2-byte values)
static uint64_t codes_bytes(uint32_t ftype, uint64_t n_blocks) { return n_blocks * (ftype == LV_Q4_0 ? 16 : 32); }

static uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Copies one GGML-format quantised tensor to `dst` (device, 256-byte aligned, matrix_device_bytes long)
// through a device staging buffer and splits it there.
static uint64_t matrix_device_bytes(uint32_t ftype, uint64_t rows, uint64_t cols, uint32_t file_version)
{
    const uint64_t nblk = rows * (cols / 32);
    return align_up(codes_bytes(ftype, nblk), 256) + align_up(nblk * (file_version == 1 ? 4 : 2), 256);
}

static int place_matrix(lv_ctx *c, lv_matrix *m, uint8_t *dst, const void *host_blocks, uint32_t ftype, uint32_t rows,
                        uint32_t cols, uint8_t *staging, uint32_t file_version)
{
    const uint64_t nblk = (uint64_t)rows * (cols / 32);
    const uint64_t raw = ggml_bytes(ftype, (uint64_t)rows * cols, file_version);
    HIP_TRY(hipMemcpyAsync(staging, host_blocks, raw, hipMemcpyHostToDevice, c->stream));
    uint4 *codes = reinterpret_cast<uint4 *>(dst);
    uint8_t *scale_plane = dst + align_up(codes_bytes(ftype, nblk), 256);
    uint16_t *scales = file_version == 1 ? nullptr : reinterpret_cast<uint16_t *>(scale_plane);
    float *scales_f32 = file_version == 1 ? reinterpret_cast<float *>(scale_plane) : nullptr;
    const unsigned grid = (unsigned)((nblk + 255) / 256);
    if (file_version == 1) {
        if (ftype == LV_Q4_0) repack_v1_kernel<4><<<dim3(grid), dim3(256), 0, c->stream>>>(staging, codes, scales_f32, nblk);
        else repack_v1_kernel<8><<<dim3(grid), dim3(256), 0, c->stream>>>(staging, codes, scales_f32, nblk);
    } else if (ftype == LV_Q4_0) {
        repack_kernel<4><<<dim3(grid), dim3(256), 0, c->stream>>>(staging, codes, scales, nblk);
    } else {
        repack_kernel<8><<<dim3(grid), dim3(256), 0, c->stream>>>(staging, codes, scales, nblk);
    }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipStreamSynchronize(c->stream));  // staging is reused by the next tensor
    m->ctx = c;
    m->view.codes = codes;
    m->view.scales = scales;
    m->view.scales_f32 = scales_f32;
    m->view.rows = rows;
    m->view.cols = cols;
    m->ftype = ftype;
    m->bytes = raw;
    return LV_OK;
}

static int check_quant_shape(const char *who, uint32_t ftype, uint32_t file_version, uint32_t rows, uint32_t cols)
{
    if (ftype != LV_Q4_0 && ftype != LV_Q8_0) return fail(LV_ERR_ARG, "%s: type %u is not q4_0/q8_0", who, ftype);
    if (file_version != 3 && file_version != 1)
        return fail(LV_ERR_ARG, "%s: file version %u (1: fp32 block scales, 3: fp16 block scales)", who, file_version);
    if (rows == 0 || cols == 0 || cols % 32) return fail(LV_ERR_ARG, "%s: shape %u x %u", who, rows, cols);
    if (cols / 32 > 768) return fail(LV_ERR_ARG, "%s: %u columns exceed the 24576 the GEMV kernels cover", who, cols);
    return LV_OK;
}

extern "C" int lv_matrix_upload(lv_ctx *c, const void *blocks, uint32_t ftype, uint32_t file_version, uint32_t rows,
                                uint32_t cols, lv_matrix **out)
{
    if (!c || !blocks || !out) return fail(LV_ERR_ARG, "lv_matrix_upload: null argument");
    *out = nullptr;
    LV_TRY(check_quant_shape("lv_matrix_upload", ftype, file_version, rows, cols));
    HIP_TRY(hipSetDevice(c->device));
    lv_matrix *m = new (std::nothrow) lv_matrix;
    if (!m) return fail(LV_ERR_OOM, "lv_matrix_upload: host allocation");
    uint8_t *staging = nullptr;
    const uint64_t raw = ggml_bytes(ftype, (uint64_t)rows * cols, file_version);
    hipError_t e = hipMalloc(&m->owned, matrix_device_bytes(ftype, rows, cols, file_version));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&staging), raw);
    int rc = LV_OK;
    if (e != hipSuccess) rc = fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "lv_matrix_upload: %s", hipGetErrorString(e));
    if (rc == LV_OK) rc = place_matrix(c, m, static_cast<uint8_t *>(m->owned), blocks, ftype, rows, cols, staging, file_version);
    (void)hipFree(staging);
    if (rc != LV_OK) {
        (void)hipFree(m->owned);
        delete m;
        return rc;
    }
    *out = m;
    return LV_OK;
}

extern "C" int lv_matrix_destroy(lv_matrix *m)
{
    if (!m) return LV_OK;
    if (m->h16_owned) {
        // launches that read the copy may still be queued on the context's stream
        if (m->ctx) { (void)hipSetDevice(m->ctx->device); (void)hipStreamSynchronize(m->ctx->stream); }
        (void)hipFree(m->h16_owned);
    }
    if (m->owned) (void)hipFree(m->owned);
    delete m;
    return LV_OK;
}

extern "C" int lv_matrix_bytes(const lv_matrix *m, uint64_t *bytes)
{
    if (!m || !bytes) return fail(LV_ERR_ARG, "lv_matrix_bytes: null argument");
    *bytes = m->bytes;
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// kernel launchers
// -----------------------------------------------------------------------------------------------------------
template <int QT, int MODE, int CW, int P>
static void launch_gemv_cfg(const GemvArgs &a, uint32_t batch, hipStream_t st)
{
    constexpr int RPW = 4;
    constexpr int rows_per_wg = (4 / CW) * RPW;
    const unsigned grid = (a.w.rows + rows_per_wg - 1) / rows_per_wg;
    gemv_kernel<QT, MODE, CW, P, RPW><<<dim3(grid, batch), dim3(256), 0, st>>>(a);
}

// matrices that can keep 256 workgroups busy go through the streaming kernel (x staged once per workgroup)
static bool gemv_streams(const MatView &w, uint32_t batch)
{
    return w.rows >= 2048 && w.cols <= (uint32_t)kWideMaxK && batch <= 8;
}

template <int QT, int MODE>
static void launch_gemv_mode(const GemvArgs &a, uint32_t batch, hipStream_t st)
{
    const uint32_t nb = a.w.cols / 32;
    if (gemv_streams(a.w, batch)) {
        const uint32_t rows_per_wg = (a.w.rows + 255) / 256;
        const uint32_t ns = (nb + 63) / 64, nr = kWideWaves / ns, per_set = (rows_per_wg + nr - 1) / nr;
        const size_t red_bytes = (size_t)per_set * nr * (MODE == kGemvSilu ? 2 : 1) * ns * sizeof(float);
        const dim3 grid((a.w.rows + rows_per_wg - 1) / rows_per_wg, batch);
        if (a.w.scales_f32) gemv_wide_kernel<QT, MODE, true><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
        else gemv_wide_kernel<QT, MODE, false><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
        return;
    }
    if (nb <= 64) launch_gemv_cfg<QT, MODE, 1, 1>(a, batch, st);
    else if (nb <= 128) launch_gemv_cfg<QT, MODE, 2, 1>(a, batch, st);
    else if (nb <= 256) launch_gemv_cfg<QT, MODE, 4, 1>(a, batch, st);
    else if (nb <= 512) launch_gemv_cfg<QT, MODE, 4, 2>(a, batch, st);
    else launch_gemv_cfg<QT, MODE, 4, 3>(a, batch, st);
}

// norm_w (optional): x is normalised inside the kernel; only valid when gemv_streams(w, batch)
static int launch_gemv(hipStream_t st, float *out, const lv_matrix &w, const lv_matrix *w1, const float *x, uint32_t batch,
                       int mode, const float *norm_w = nullptr)
{
    GemvArgs a{};
    a.w = w.view;
    if (w1) a.w1 = w1->view;
    if (w1 && (w1->view.scales_f32 != nullptr) != (w.view.scales_f32 != nullptr))
        return fail(LV_ERR_ARG, "gemv: the two matrices come from different file versions (fp16 and fp32 block scales)");
    a.x = x;
    a.out = out;
    a.norm_w = norm_w;
    if (norm_w && !gemv_streams(a.w, batch)) return fail(LV_ERR_ARG, "gemv: fused normalisation needs the streaming kernel");
    const bool q4 = w.ftype == LV_Q4_0;
    switch (mode) {
    case kGemvStore: q4 ? launch_gemv_mode<4, kGemvStore>(a, batch, st) : launch_gemv_mode<8, kGemvStore>(a, batch, st); break;
    case kGemvAdd: q4 ? launch_gemv_mode<4, kGemvAdd>(a, batch, st) : launch_gemv_mode<8, kGemvAdd>(a, batch, st); break;
    default: q4 ? launch_gemv_mode<4, kGemvSilu>(a, batch, st) : launch_gemv_mode<8, kGemvSilu>(a, batch, st); break;
    }
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// Three same-shape matrices applied to one vector (the q, k and v projections of a token) as one launch when the
// streaming kernel covers the shape, else as three.
struct Gemv3Extras {
    const float *norm_w = nullptr;                 // normalise x inside the kernel
    uint16_t *cache[3] = {nullptr, nullptr, nullptr};  // append result i to this cache plane as fp16
    const uint32_t *pos_ptr = nullptr;
    uint32_t pos_add = 0, backlog = 0;
};
static bool gemv3_streams(const lv_matrix *const w[3])
{
    const lv_matrix &w0 = *w[0];
    bool same = true;
    for (int i = 1; i < 3; i++)
        same = same && w[i]->ftype == w0.ftype && w[i]->view.rows == w0.view.rows && w[i]->view.cols == w0.view.cols &&
               (w[i]->view.scales_f32 != nullptr) == (w0.view.scales_f32 != nullptr);
    return same && gemv_streams(w0.view, 1);
}
static int launch_gemv3(hipStream_t st, float *const out[3], const lv_matrix *const w[3], const float *x, const Gemv3Extras *ex = nullptr)
{
    const lv_matrix &w0 = *w[0];
    if (gemv3_streams(w)) {
        GemvArgs3 a{};
        for (int i = 0; i < 3; i++) {
            a.m[i].w = w[i]->view; a.m[i].x = x; a.m[i].out = out[i];
            if (ex) {
                a.m[i].norm_w = ex->norm_w; a.m[i].cache = ex->cache[i]; a.m[i].pos_ptr = ex->pos_ptr; a.m[i].pos_add = ex->pos_add;
                a.m[i].backlog = ex->backlog;
            }
        }
        const uint32_t rows = w0.view.rows, nb = w0.view.cols / 32;
        const uint32_t rows_per_wg = (rows + 255) / 256;
        const uint32_t ns = (nb + 63) / 64, nr = kWideWaves / ns, per_set = (rows_per_wg + nr - 1) / nr;
        const size_t red_bytes = (size_t)per_set * nr * ns * sizeof(float);
        const dim3 grid((rows + rows_per_wg - 1) / rows_per_wg, 3);
        const bool sf32 = w0.view.scales_f32 != nullptr;
        if (w0.ftype == LV_Q4_0) {
            if (sf32) gemv_wide3_kernel<4, true><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
            else gemv_wide3_kernel<4, false><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
        } else {
            if (sf32) gemv_wide3_kernel<8, true><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
            else gemv_wide3_kernel<8, false><<<grid, dim3(kWideWaves * 64), red_bytes, st>>>(a, rows_per_wg);
        }
        HIP_TRY(hipGetLastError());
        return LV_OK;
    }
    if (ex) return fail(LV_ERR_ARG, "gemv3: fused extras need the streaming kernel");
    for (int i = 0; i < 3; i++) LV_TRY(launch_gemv(st, out[i], *w[i], nullptr, x, 1, kGemvStore));
    return LV_OK;
}

constexpr uint32_t kPrefillMin = 16;       // below this the rows of a step go through the one-token kernels

static size_t attn_part_floats(uint32_t batch, uint32_t heads, uint32_t splits, uint32_t rot)
{
    return (size_t)batch * heads * splits * (rot + 1);
}

static int launch_attention(hipStream_t st, float *out, const uint16_t *kc, const uint16_t *vc, const float *q,
                            const float2 *trig, float *part, uint32_t *counters, const uint32_t *pos_ptr, uint32_t pos_add,
                            uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch)
{
    AttnArgs a{};
    a.out = out; a.kcache = kc; a.vcache = vc; a.q = q; a.trig = trig; a.part = part; a.counters = counters;
    a.pos_ptr = pos_ptr; a.pos_add = pos_add; a.heads = heads; a.backlog = backlog; a.chunk = kAttnChunk;
    a.splits = (backlog + kAttnChunk - 1) / kAttnChunk;
    const dim3 grid(heads, a.splits, batch);
    const size_t lds = sizeof(float) * 4 * (rot + 1);
    switch (rot) {
    case 32: attention_kernel<32><<<grid, dim3(256), lds, st>>>(a); break;
    case 64: attention_kernel<64><<<grid, dim3(256), lds, st>>>(a); break;
    case 128: attention_kernel<128><<<grid, dim3(256), lds, st>>>(a); break;
    default: return fail(LV_ERR_ARG, "attention: head size %u (32, 64 and 128 are built)", rot);
    }
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// Batched (prompt) attention of one layer: the operand planes of positions 0 .. pos + n - 1, then the attention kernel.
// `planes`: four planes of attn_plane_halfs(backlog, heads, rot) halfs.  kin / vin: the batch's K and V rows, not yet in the cache
// (the first kernel appends them), or null when the cache already holds them.  The result goes to `out` (fp32 rows) and/or to the
// activation halves xh / xl (tile order, width Kp; the rows up to the next multiple of 128 are written as zeros).
static int launch_attention_batch(hipStream_t st, float *out, uint16_t *xh, uint16_t *xl, uint32_t Kp, uint16_t *planes, uint16_t *kc,
                                  uint16_t *vc, const float *kin, const float *vin, const float *q, const float2 *trig_abs, const uint32_t *pos_ptr, uint32_t pos_add, uint32_t n,
                                  uint32_t backlog, uint32_t heads, uint32_t rot)
{
    const size_t ph = attn_plane_halfs(backlog, heads, rot);
    AttnPrepArgs p{};
    p.pl.kh = planes; p.pl.kl = planes + ph; p.pl.v1 = planes + 2 * ph; p.pl.v2 = planes + 3 * ph;
    p.kcache = kc; p.vcache = vc; p.kin = kin; p.vin = vin; p.trig_abs = trig_abs; p.pos_ptr = pos_ptr; p.pos_add = pos_add; p.n = n; p.heads = heads; p.backlog = backlog;
    AttnBatchArgs a{};
    a.out = out; a.xh = xh; a.xl = xl; a.Kp = Kp; a.pl = p.pl; a.q = q; a.trig_abs = trig_abs; a.pos_ptr = pos_ptr; a.pos_add = pos_add;
    a.n = n; a.heads = heads; a.backlog = backlog;
    const dim3 pgrid(heads, attn_rows64(backlog) / kAttnBatchK);
    const uint32_t n_pad = xh ? (n + kGemmTile - 1) / kGemmTile * kGemmTile : n;
    const dim3 grid(heads, (n_pad + kAttnBatchQ - 1) / kAttnBatchQ);
    const size_t lds = (size_t)1024 * rot;
    // more than 64 KB of dynamic LDS has to be allowed per function, on the device that launches it
#define LV_ATTN_BATCH(R)                                                                                                              \
    case R:                                                                                                                           \
        attention_prepare_kernel<R><<<pgrid, dim3(256), 0, st>>>(p);                                                                  \
        HIP_TRY(hipGetLastError());                                                                                                   \
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_batch_kernel<R>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        attention_batch_kernel<R><<<grid, dim3(256), lds, st>>>(a);                                                                   \
        break;
    switch (rot) {
        LV_ATTN_BATCH(32)
        LV_ATTN_BATCH(64)
        LV_ATTN_BATCH(128)
    default: return fail(LV_ERR_ARG, "attention: head size %u (32, 64 and 128 are built)", rot);
    }
#undef LV_ATTN_BATCH
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// cos/sin of delta*theta_i with the argument rounded the way mhsa.comp:45 rounds it:
// theta_i = pow(10000, -i/(R/2)) in fp32, delta*theta_i as one fp32 product.
static void build_trig(std::vector<float2> &t, uint32_t rows, uint32_t rot)
{
    const uint32_t half = rot / 2;
    t.resize((size_t)rows * half);
    std::vector<float> freq(half);
    for (uint32_t i = 0; i < half; i++) freq[i] = powf(10000.0f, -(float)i / (float)half);
    for (uint32_t d = 0; d < rows; d++)
        for (uint32_t i = 0; i < half; i++) {
            const float ang = (float)d * freq[i];
            t[(size_t)d * half + i] = make_float2((float)cos((double)ang), (float)sin((double)ang));
        }
}

// cos/sin of p * theta_i for the batched attention, which rotates rows by their absolute position: theta_i rounded to
// fp32 as above, the product and the functions in double (the difference of two such angles then differs from the
// shader's fp32-rounded delta * theta_i by that one rounding only)
static void build_trig_abs(std::vector<float2> &t, uint32_t rows, uint32_t rot)
{
    const uint32_t half = rot / 2;
    t.resize((size_t)rows * half);
    for (uint32_t i = 0; i < half; i++) {
        const double freq = (double)powf(10000.0f, -(float)i / (float)half);
        for (uint32_t d = 0; d < rows; d++) {
            const double ang = (double)d * freq;
            t[(size_t)d * half + i] = make_float2((float)cos(ang), (float)sin(ang));
        }
    }
}

static int upload_trig(float2 **dev, uint32_t rows, uint32_t rot, hipStream_t st, bool absolute = false)
{
    std::vector<float2> t;
    if (absolute) build_trig_abs(t, rows, rot);
    else build_trig(t, rows, rot);
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(dev), t.size() * sizeof(float2)));
    HIP_TRY(hipMemcpyAsync(*dev, t.data(), t.size() * sizeof(float2), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// single-kernel entry points
// -----------------------------------------------------------------------------------------------------------
extern "C" int lv_kernel_dequant(lv_ctx *c, const lv_matrix *m, uint32_t row0, uint32_t n_rows, float *dst)
{
    if (!c || !m || !dst) return fail(LV_ERR_ARG, "lv_kernel_dequant: null argument");
    if ((uint64_t)row0 + n_rows > m->view.rows) return fail(LV_ERR_RANGE, "lv_kernel_dequant: rows %u+%u of %u", row0, n_rows, m->view.rows);
    if (n_rows == 0) return LV_OK;
    const uint64_t nb = m->view.cols / 32, first = (uint64_t)row0 * nb, count = (uint64_t)n_rows * nb;
    const unsigned grid = (unsigned)((count + 255) / 256);
    if (m->ftype == LV_Q4_0) dequant_kernel<4><<<dim3(grid), dim3(256), 0, c->stream>>>(m->view, first, count, dst);
    else dequant_kernel<8><<<dim3(grid), dim3(256), 0, c->stream>>>(m->view, first, count, dst);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

extern "C" int lv_kernel_gemv(lv_ctx *c, float *out, const lv_matrix *w, const float *x, uint32_t batch, int accumulate)
{
    if (!c || !out || !w || !x) return fail(LV_ERR_ARG, "lv_kernel_gemv: null argument");
    if (batch == 0) return LV_OK;
    if (batch > 65535) return fail(LV_ERR_RANGE, "lv_kernel_gemv: batch %u", batch);
    return launch_gemv(c->stream, out, *w, nullptr, x, batch, accumulate ? kGemvAdd : kGemvStore);
}

extern "C" int lv_kernel_gemv_silu(lv_ctx *c, float *out, const lv_matrix *w3, const lv_matrix *w1, const float *x, uint32_t batch)
{
    if (!c || !out || !w3 || !w1 || !x) return fail(LV_ERR_ARG, "lv_kernel_gemv_silu: null argument");
    if (w3->ftype != w1->ftype || w3->view.rows != w1->view.rows || w3->view.cols != w1->view.cols)
        return fail(LV_ERR_ARG, "lv_kernel_gemv_silu: the two matrices differ in type or shape");
    if (batch == 0) return LV_OK;
    if (batch > 65535) return fail(LV_ERR_RANGE, "lv_kernel_gemv_silu: batch %u", batch);
    return launch_gemv(c->stream, out, *w3, w1, x, batch, kGemvSilu);
}

// out[n][ldo] (+)= x[n][K] * W^T on the matrix cores; xh/xl = workspace for the fp16 halves of x, n_pad rows
static int launch_gemm_presplit(hipStream_t st, float *out, uint32_t ldo, const lv_matrix &w, uint32_t n, const uint16_t *xh, const uint16_t *xl,
                                bool accumulate, const float *xscale = nullptr);

// fp32 activations -> the two fp16 halves the GEMM multiplies; with xscale, scaled row by row (inputs of unknown size)
static int launch_split(hipStream_t st, uint16_t *xh, uint16_t *xl, float *xscale, const float *x, uint32_t n, uint32_t K)
{
    const uint32_t n_pad = (n + kGemmTile - 1) / kGemmTile * kGemmTile, Kp = gemm_k_padded(K);
    if (K % 8) return fail(LV_ERR_ARG, "gemm: %u columns", K);
    if (!xscale) split_half_kernel<<<dim3(Kp / 64, n_pad / 32), dim3(256), 0, st>>>(xh, xl, x, n, K, Kp);
    else if (Kp <= 2048 * 3) split_rows_kernel<3><<<dim3(n_pad), dim3(256), 0, st>>>(xh, xl, xscale, x, n, K, Kp);
    else if (Kp <= 2048 * 7) split_rows_kernel<7><<<dim3(n_pad), dim3(256), 0, st>>>(xh, xl, xscale, x, n, K, Kp);
    else split_rows_kernel<0><<<dim3(n_pad), dim3(256), 0, st>>>(xh, xl, xscale, x, n, K, Kp);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// the prompt copy of one matrix into dst (gemm_copy_halfs halfs)
static uint64_t prompt_copy_halfs(const lv_matrix &w) { return gemm_copy_halfs(w.view.rows, w.view.cols); }
static int launch_expand(hipStream_t st, uint16_t *dst, const lv_matrix &w)
{
    const uint64_t threads = (uint64_t)gemm_rows_padded(w.view.rows) * (gemm_k_padded(w.view.cols) / 32);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (w.ftype == LV_Q4_0) expand_codes_kernel<4, false><<<grid, dim3(256), 0, st>>>(dst, w.view, w.view);
    else if (w.ftype == LV_Q8_0) expand_codes_kernel<8, false><<<grid, dim3(256), 0, st>>>(dst, w.view, w.view);
    else return fail(LV_ERR_ARG, "gemm: matrix type %u", w.ftype);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// The feed-forward's gate (W3) and up (W1) matrices as one pair copy (expand_codes_kernel<.., true>), whose GEMM applies
// SwiGLU in its epilogue.  Possible when the two have one shape, type and kind of scale plane and 128 divides their rows.
static bool gemm_same(const lv_matrix &a, const lv_matrix &b);
static bool gemm_pairable(const lv_matrix &gate, const lv_matrix &up)
{
    return gemm_same(gate, up) && gate.view.rows % 128 == 0 && (gate.ftype == LV_Q4_0 || gate.ftype == LV_Q8_0);
}
static uint64_t pair_copy_halfs(const lv_matrix &gate) { return gemm_copy_halfs(2 * gate.view.rows, gate.view.cols); }
static int launch_expand_pair(hipStream_t st, uint16_t *dst, const lv_matrix &gate, const lv_matrix &up)
{
    const uint64_t threads = (uint64_t)gemm_rows_padded(2 * gate.view.rows) * (gemm_k_padded(gate.view.cols) / 32);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (gate.ftype == LV_Q4_0) expand_codes_kernel<4, true><<<grid, dim3(256), 0, st>>>(dst, gate.view, up.view);
    else expand_codes_kernel<8, true><<<grid, dim3(256), 0, st>>>(dst, gate.view, up.view);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// launches gemm_kernel for args whose w16[0..nz-1] and outs[0..nz-1] are set: nz matrices of one shape, or nz K slices of one
static int dispatch_gemm(hipStream_t st, GemmArgs a, const lv_matrix &w, uint32_t nz)
{
    a.rows = w.view.rows; a.K = w.view.cols;
    for (uint32_t i = 0; i < nz; i++)
        if (!a.w16[i]) return fail(LV_ERR_STATE, "gemm: the matrix has no prompt copy");
    // 132 KB of dynamic LDS need the attribute on the device the launch goes to; setting it is a host-side table entry
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLdsBytes));
    const uint32_t token_tiles = (a.n + kGemmTile - 1) / kGemmTile, row_tiles = (a.rows + kGemmRows - 1) / kGemmRows;
    a.nz = nz;
    const dim3 grid((row_tiles * nz + 7) / 8 * 8 * token_tiles);
    gemm_kernel<false><<<grid, dim3(512), kGemmLdsBytes, st>>>(a);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// q, k and v of a prompt batch (three matrices of one shape) as one launch: q as fp32 rows of `q`, k and v rounded to fp16
// straight into rows *row_ptr + row_add .. of their caches (rows of `dim` halfs, `backlog` of them)
static int launch_gemm_qkv(hipStream_t st, float *q, uint16_t *kcache, uint16_t *vcache, const lv_matrix &wq, const lv_matrix &wk, const lv_matrix &wv,
                           uint32_t n, const uint16_t *xh, const uint16_t *xl, const float *xscale, const uint32_t *row_ptr, uint32_t row_add,
                           uint32_t backlog)
{
    GemmArgs a{};
    a.xh = xh; a.xl = xl; a.n = n; a.xscale = xscale; a.rows = wq.view.rows; a.K = wq.view.cols; a.nz = 3; a.ldo = wq.view.rows;
    a.outs[0] = q; a.w16[0] = wq.h16; a.w16[1] = wk.h16; a.w16[2] = wv.h16;
    a.half_out[1] = kcache; a.half_out[2] = vcache; a.row_ptr = row_ptr; a.row_add = row_add; a.row_limit = backlog;
    for (int i = 0; i < 3; i++)
        if (!a.w16[i]) return fail(LV_ERR_STATE, "gemm: the matrix has no prompt copy");
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_rows16_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLdsBytes));
    const uint32_t token_tiles = (n + kGemmTile - 1) / kGemmTile, row_tiles = (a.rows + kGemmRows - 1) / kGemmRows;
    const dim3 grid((row_tiles * 3 + 7) / 8 * 8 * token_tiles);
    gemm_rows16_kernel<<<grid, dim3(512), kGemmLdsBytes, st>>>(a);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// fh, fl (tile order, n_pad x gemm_k_padded(F)) = the halves of SwiGLU(x W3^T, x W1^T) for the pair copy `pair16` of two F x K matrices.
// Rounds.  A round holds 32 workgroups per XCD, i.e. cap = (32 / token tiles) * 8 row tiles.  When the last round would be
// less than half full (7B at 512 tokens: 86 row tiles, 64 a round, 22 left) its row tiles are cut in two along K instead
// and run as ONE round of half the length: raw products of both halves into g1 / g2 (scratch, n_pad x F floats each), summed
// and passed through SwiGLU by silu_pair_tail_kernel.
static int launch_gemm_silu(hipStream_t st, uint16_t *fh, uint16_t *fl, const uint16_t *pair16, uint32_t F, uint32_t K, uint32_t n,
                            const uint16_t *xh, const uint16_t *xl, const float *xscale, float *g1, float *g2)
{
    const uint32_t token_tiles = (n + kGemmTile - 1) / kGemmTile, tiles = 2 * F / kGemmRows, k_steps = gemm_k_padded(K) / kGemmK;
    const uint32_t cap = token_tiles <= 32 ? (32 / token_tiles) * 8 : 0;
    uint32_t tail = cap ? tiles % cap : 0;
    if (tiles < cap + tail || tail * 2 > cap || k_steps < 32 || k_steps % 2 || !g1 || !g2) tail = 0;
    const uint32_t head = tiles - tail;
    GemmArgs a{};
    a.xh = xh; a.xl = xl; a.n = n; a.xscale = xscale; a.w16[0] = pair16; a.rows = 2 * F; a.K = K; a.nz = 1;
    a.fh = fh; a.fl = fl; a.fKp = gemm_k_padded(F);
    a.tile0 = 0; a.tile_count = head;
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLdsBytes));
    gemm_kernel<true><<<dim3((head + 7) / 8 * 8 * token_tiles), dim3(512), kGemmLdsBytes, st>>>(a);
    HIP_TRY(hipGetLastError());
    if (!tail) return LV_OK;
    GemmArgs b{};
    b.xh = xh; b.xl = xl; b.n = n; b.xscale = xscale; b.rows = 2 * F; b.K = K; b.nz = 2;
    b.w16[0] = b.w16[1] = pair16; b.outs[0] = g1; b.outs[1] = g2; b.ldo = tail * kGemmRows;
    b.slice_k = k_steps / 2 * kGemmK; b.tile0 = head; b.tile_count = tail;
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLdsBytes));
    gemm_kernel<false><<<dim3((tail * 2 + 7) / 8 * 8 * token_tiles), dim3(512), kGemmLdsBytes, st>>>(b);
    HIP_TRY(hipGetLastError());
    SiluTailArgs t{};
    t.fh = fh; t.fl = fl; t.parts[0] = g1; t.parts[1] = g2; t.nparts = 2; t.n = n; t.F = F; t.Fp = gemm_k_padded(F); t.f0 = head * (kGemmRows / 2);
    t.tail_rows = tail * kGemmRows;
    silu_pair_tail_kernel<<<dim3((F - t.f0) / 64, token_tiles * kGemmTile / 32), dim3(256), 0, st>>>(t);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// the same with the activations already split (one split serves wq, wk, wv or w3, w1); nmat matrices of one shape,
// type and scale plane as one launch
static int launch_gemm_multi(hipStream_t st, float *const outs[], uint32_t ldo, const lv_matrix *const ws[], int nmat, uint32_t n,
                             const uint16_t *xh, const uint16_t *xl, bool accumulate, const float *xscale = nullptr)
{
    GemmArgs a{};
    a.xscale = xscale;
    for (int i = 0; i < nmat; i++) { a.outs[i] = outs[i]; a.w16[i] = ws[i]->h16; }
    a.xh = xh; a.xl = xl; a.n = n; a.ldo = ldo; a.accumulate = accumulate ? 1 : 0;
    return dispatch_gemm(st, a, *ws[0], (uint32_t)nmat);
}

// Into how many K slices (1..4) to cut a product of `row_tiles` x `token_tiles` output tiles over `k_steps` steps of 64.
// gemm_kernel deals (slice, row tile) units to the 8 XCDs in turn, each unit's token tiles to CUs of its XCD (32 a
// round); the cost of a choice is its rounds times the steps of a slice, plus two steps per extra slice for the pass
// that adds the slices up.  A slice keeps at least 16 steps.
static uint32_t gemm_k_slices(uint32_t row_tiles, uint32_t token_tiles, uint32_t k_steps)
{
    uint32_t best = 1, best_cost = ~0u;
    for (uint32_t s = 1; s <= (uint32_t)kGemmMaxMats; s++) {
        if (s > 1 && k_steps / s < 16) break;
        const uint32_t per_xcd = (row_tiles * s + 7) / 8 * token_tiles, rounds = (per_xcd + 31) / 32;
        const uint32_t cost = rounds * ((k_steps + s - 1) / s) + 2 * (s - 1);
        if (cost < best_cost) { best_cost = cost; best = s; }
    }
    return best;
}

// out[n][ldo] (+)= the sum of `count` K slices [n][rows]
static int launch_gemm_reduce(hipStream_t st, float *out, uint32_t ldo, float *const parts[kGemmMaxMats], uint32_t count, uint32_t rows, uint32_t n,
                              bool accumulate)
{
    GemmReduceArgs r{};
    for (uint32_t i = 0; i < count; i++) r.parts[i] = parts[i];
    r.out = out; r.nparts = count; r.rows = rows; r.ldo = ldo; r.n = n; r.accumulate = accumulate ? 1 : 0;
    gemm_reduce_kernel<<<dim3((rows / 4 + 255) / 256, n), dim3(256), 0, st>>>(r);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

// the slice count launch_gemm_sliced uses for n tokens of w into rows of ldo floats (the reduce works on float4)
static uint32_t gemm_slices_for(const lv_matrix &w, uint32_t n, uint32_t ldo)
{
    const uint32_t rows = w.view.rows, k_steps = (w.view.cols + kGemmK - 1) / kGemmK;
    const uint32_t token_tiles = (n + kGemmTile - 1) / kGemmTile;
    return (rows % 4 || ldo % 4) ? 1 : gemm_k_slices((rows + kGemmRows - 1) / kGemmRows, token_tiles, k_steps);
}

// one matrix, activations already split, K cut in slices when that fills the CUs better: the slices go to parts[]
// ([n][rows] floats each, scratch of the caller) and gemm_reduce_kernel adds them to out in a fixed order
// With `pending` given, the slices are left unsummed and *pending says how many there are (0: out is complete): the
// caller adds them to out itself (prefill_norm_kernel does, on its way through the row).
static int launch_gemm_sliced(hipStream_t st, float *out, uint32_t ldo, const lv_matrix &w, uint32_t n, const uint16_t *xh, const uint16_t *xl,
                              const float *xscale, bool accumulate, float *const parts[kGemmMaxMats], uint32_t *pending = nullptr)
{
    if (pending) *pending = 0;
    const uint32_t rows = w.view.rows, k_steps = (w.view.cols + kGemmK - 1) / kGemmK;
    const uint32_t slices = parts ? gemm_slices_for(w, n, ldo) : 1;
    GemmArgs a{};
    a.xh = xh; a.xl = xl; a.n = n; a.xscale = xscale;
    if (slices == 1) {
        a.outs[0] = out; a.w16[0] = w.h16; a.ldo = ldo; a.accumulate = accumulate ? 1 : 0;
        return dispatch_gemm(st, a, w, 1);
    }
    const uint32_t slice_steps = (k_steps + slices - 1) / slices;
    a.slice_k = slice_steps * kGemmK;
    const uint32_t used = (k_steps + slice_steps - 1) / slice_steps;      // every slice launched has a step
    for (uint32_t i = 0; i < used; i++) { a.outs[i] = parts[i]; a.w16[i] = w.h16; }
    a.ldo = rows;
    LV_TRY(dispatch_gemm(st, a, w, used));
    if (pending && accumulate) { *pending = used; return LV_OK; }
    return launch_gemm_reduce(st, out, ldo, parts, used, rows, n, accumulate);
}

static int launch_gemm_presplit(hipStream_t st, float *out, uint32_t ldo, const lv_matrix &w, uint32_t n, const uint16_t *xh, const uint16_t *xl,
                                bool accumulate, const float *xscale)
{
    float *const outs[1] = {out};
    const lv_matrix *const ws[1] = {&w};
    return launch_gemm_multi(st, outs, ldo, ws, 1, n, xh, xl, accumulate, xscale);
}

// can these matrices share a launch?  (one shape, one type, one kind of scale plane)
static bool gemm_same(const lv_matrix &a, const lv_matrix &b)
{
    return a.ftype == b.ftype && a.view.rows == b.view.rows && a.view.cols == b.view.cols && (a.view.scales_f32 != nullptr) == (b.view.scales_f32 != nullptr);
}

extern "C" int lv_kernel_gemm(lv_ctx *c, float *out, const lv_matrix *w, const float *x, uint32_t batch, int accumulate)
{
    if (!c || !out || !w || !x) return fail(LV_ERR_ARG, "lv_kernel_gemm: null argument");
    if (batch == 0) return LV_OK;
    if (batch > kMaxStepTokens) return fail(LV_ERR_RANGE, "lv_kernel_gemm: batch %u (limit %u)", batch, kMaxStepTokens);
    HIP_TRY(hipSetDevice(c->device));
    const size_t n_pad = (batch + kGemmTile - 1) / kGemmTile * kGemmTile, halfs = n_pad * gemm_k_padded(w->view.cols);
    if (w->view.cols % 32) return fail(LV_ERR_ARG, "gemm: %u columns", w->view.cols);
    // the copy made below is freed by lv_matrix_destroy after a wait for the matrix's own context
    if (!w->h16 && w->ctx != c) return fail(LV_ERR_ARG, "lv_kernel_gemm: the matrix belongs to another context");
    // The matrix's prompt copy is made by the first call and stays with the matrix; the workspace (the two fp16 halves of
    // the activations, their row scales and, where K is cut in slices, the partial results) stays with the context.
    if (!w->h16) {
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->h16_owned), (size_t)prompt_copy_halfs(*w) * 2);
        if (e != hipSuccess) { w->h16_owned = nullptr; return fail(LV_ERR_OOM, "lv_kernel_gemm: prompt copy of the matrix"); }
        int rc = launch_expand(c->stream, w->h16_owned, *w);
        if (rc != LV_OK) {
            (void)hipStreamSynchronize(c->stream);
            (void)hipFree(w->h16_owned);
            w->h16_owned = nullptr;
            return rc;
        }
        w->h16 = w->h16_owned;
    }
    const uint32_t slices = gemm_slices_for(*w, batch, w->view.rows);
    const size_t part = slices > 1 ? (size_t)batch * w->view.rows : 0;
    const size_t need = halfs * 2 * 2 + n_pad * 4 + part * slices * 4;
    if (need > c->gemm_ws_bytes) {
        HIP_TRY(hipStreamSynchronize(c->stream));
        (void)hipFree(c->gemm_ws);
        c->gemm_ws = nullptr;
        c->gemm_ws_bytes = 0;
        if (hipMalloc(reinterpret_cast<void **>(&c->gemm_ws), need) != hipSuccess) {
            c->gemm_ws = nullptr;
            return fail(LV_ERR_OOM, "lv_kernel_gemm: workspace");
        }
        c->gemm_ws_bytes = need;
    }
    uint16_t *xh = c->gemm_ws, *xl = xh + halfs;
    float *xscale = reinterpret_cast<float *>(xl + halfs);
    float *p0 = xscale + n_pad;
    float *const parts[kGemmMaxMats] = {p0, p0 + part, p0 + 2 * part, p0 + 3 * part};
    LV_TRY(launch_split(c->stream, xh, xl, xscale, x, batch, w->view.cols));
    return launch_gemm_sliced(c->stream, out, w->view.rows, *w, batch, xh, xl, xscale, accumulate != 0, slices > 1 ? parts : nullptr);
}

extern "C" int lv_kernel_normalize(lv_ctx *c, float *out, const float *x, const float *w, uint32_t dim, uint32_t batch)
{
    if (!c || !out || !x || !w) return fail(LV_ERR_ARG, "lv_kernel_normalize: null argument");
    if (dim == 0) return fail(LV_ERR_ARG, "lv_kernel_normalize: dim is 0");
    if (batch == 0) return LV_OK;
    normalize_kernel<<<dim3(batch), dim3(256), 0, c->stream>>>(out, x, w, dim);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

extern "C" int lv_kernel_kv_append(lv_ctx *c, void *cache, const float *in, uint32_t pos, uint32_t dim, uint32_t batch,
                                   uint32_t backlog)
{
    if (!c || !cache || !in) return fail(LV_ERR_ARG, "lv_kernel_kv_append: null argument");
    if ((uint64_t)pos + batch > backlog) return fail(LV_ERR_RANGE, "lv_kernel_kv_append: rows %u+%u of %u", pos, batch, backlog);
    if (batch == 0 || dim == 0) return LV_OK;
    kv_append_kernel<<<dim3((dim + 255) / 256, batch), dim3(256), 0, c->stream>>>(static_cast<uint16_t *>(cache), in, nullptr,
                                                                                    pos, dim, backlog);
    HIP_TRY(hipGetLastError());
    return LV_OK;
}

extern "C" int lv_kernel_attention(lv_ctx *c, float *out, const void *kcache, const void *vcache, const float *q, uint32_t pos,
                                   uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch)
{
    if (!c || !out || !kcache || !vcache || !q) return fail(LV_ERR_ARG, "lv_kernel_attention: null argument");
    if (heads == 0 || batch == 0 || backlog == 0) return fail(LV_ERR_ARG, "lv_kernel_attention: empty shape");
    if ((uint64_t)pos + batch > backlog) return fail(LV_ERR_RANGE, "lv_kernel_attention: rows %u+%u of %u", pos, batch, backlog);
    if (rot != 32 && rot != 64 && rot != 128) return fail(LV_ERR_ARG, "lv_kernel_attention: head size %u", rot);
    HIP_TRY(hipSetDevice(c->device));
    if (batch >= kPrefillMin) {    // the kernels a prompt batch goes through
        if (c->trig_abs_rot != rot || c->trig_abs_rows < backlog) {
            HIP_TRY(hipStreamSynchronize(c->stream));
            (void)hipFree(c->trig_abs);
            c->trig_abs = nullptr;
            c->trig_abs_rows = c->trig_abs_rot = 0;
            LV_TRY(upload_trig(&c->trig_abs, backlog, rot, c->stream, true));
            c->trig_abs_rows = backlog;
            c->trig_abs_rot = rot;
        }
        const size_t planes = 4 * attn_plane_halfs(backlog, heads, rot);
        if (c->attn_plane_halfs < planes) {
            HIP_TRY(hipStreamSynchronize(c->stream));
            (void)hipFree(c->attn_planes);
            c->attn_planes = nullptr;
            c->attn_plane_halfs = 0;
            HIP_TRY(hipMalloc(reinterpret_cast<void **>(&c->attn_planes), planes * 2));
            c->attn_plane_halfs = planes;
        }
        return launch_attention_batch(c->stream, out, nullptr, nullptr, 0, c->attn_planes, static_cast<uint16_t *>(const_cast<void *>(kcache)),
                                      static_cast<uint16_t *>(const_cast<void *>(vcache)), nullptr, nullptr, q, c->trig_abs, nullptr, pos, batch, backlog, heads, rot);
    }
    if (c->trig_rot != rot || c->trig_rows < backlog) {
        HIP_TRY(hipStreamSynchronize(c->stream));
        (void)hipFree(c->trig);
        c->trig = nullptr;
        c->trig_rows = c->trig_rot = 0;
        LV_TRY(upload_trig(&c->trig, backlog, rot, c->stream));
        c->trig_rows = backlog;
        c->trig_rot = rot;
    }
    const uint32_t splits = (backlog + kAttnChunk - 1) / kAttnChunk;
    const size_t need_part = attn_part_floats(batch, heads, splits, rot), need_cnt = (size_t)batch * heads;
    if (c->attn_part_floats < need_part) {
        HIP_TRY(hipStreamSynchronize(c->stream));
        (void)hipFree(c->attn_part);
        c->attn_part = nullptr;
        c->attn_part_floats = 0;
        HIP_TRY(hipMalloc(reinterpret_cast<void **>(&c->attn_part), need_part * sizeof(float)));
        c->attn_part_floats = need_part;
    }
    if (c->attn_counter_words < need_cnt) {
        HIP_TRY(hipStreamSynchronize(c->stream));
        (void)hipFree(c->attn_counters);
        c->attn_counters = nullptr;
        c->attn_counter_words = 0;
        HIP_TRY(hipMalloc(reinterpret_cast<void **>(&c->attn_counters), need_cnt * 4));
        c->attn_counter_words = need_cnt;
        LV_TRY(zero_async(c->attn_counters, need_cnt * 4, c->stream));
    }
    return launch_attention(c->stream, out, static_cast<const uint16_t *>(kcache), static_cast<const uint16_t *>(vcache), q,
                            c->trig, c->attn_part, c->attn_counters, nullptr, pos, backlog, heads, rot, batch);
}

// cos/sin table of build_trig computed on the device (same fp32 angle rounding: theta_i from the host's powf, the
// product in fp32, the functions in double)
struct TrigFreq { float f[64]; };
__global__ void trig_fill_kernel(float2 *__restrict__ t, TrigFreq fr, uint32_t rows, uint32_t half)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * half) return;
    const uint32_t d = i / half, j = i % half;
    const float ang = (float)d * fr.f[j];
    t[i] = make_float2((float)cos((double)ang), (float)sin((double)ang));
}

// lv_kernel_attention without a single allocation: rotation table, partial sums and split counters live in this
// device's copy of the file-scope scratch array.  Calls on one device share that array, so two of them must not overlap
// (calls on one context are ordered by its stream).  The array keeps the last call's contents: the counters are cleared
// and the table rewritten by small kernels in front of the attention kernel; the partial sums are written before read.
extern "C" int lv_kernel_attention_static(lv_ctx *c, float *out, const void *kcache, const void *vcache, const float *q, uint32_t pos,
                                          uint32_t backlog, uint32_t heads, uint32_t rot, uint32_t batch)
{
    if (!c || !out || !kcache || !vcache || !q) return fail(LV_ERR_ARG, "lv_kernel_attention_static: null argument");
    if (heads == 0 || batch == 0 || backlog == 0) return fail(LV_ERR_ARG, "lv_kernel_attention_static: empty shape");
    if ((uint64_t)pos + batch > backlog) return fail(LV_ERR_RANGE, "lv_kernel_attention_static: rows %u+%u of %u", pos, batch, backlog);
    if (rot != 32 && rot != 64 && rot != 128) return fail(LV_ERR_ARG, "lv_kernel_attention_static: head size %u", rot);
    if (!c->scratch) return fail(LV_ERR_STATE, "lv_kernel_attention_static: the context has no scratch address");
    const uint64_t splits = ((uint64_t)backlog + kAttnChunk - 1) / kAttnChunk;
    const uint64_t need_trig = (uint64_t)backlog * (rot / 2), need_part = (uint64_t)batch * heads * splits * (rot + 1),
                   need_cnt = (uint64_t)batch * heads;
    if (need_trig > kStaticTrigPairs || need_part > kStaticPartFloats || need_cnt > kStaticCounters)
        return fail(LV_ERR_RANGE,
                    "lv_kernel_attention_static: backlog %u x heads %u x head size %u x batch %u exceeds the static work area "
                    "(backlog * rot / 2 <= %u, batch * heads * ceil(backlog / 64) * (rot + 1) <= %u, batch * heads <= %u)",
                    backlog, heads, rot, batch, kStaticTrigPairs, kStaticPartFloats, kStaticCounters);
    HIP_TRY(hipSetDevice(c->device));
    AttnScratch *sc = c->scratch;
    TrigFreq fr{};
    const uint32_t half = rot / 2;
    for (uint32_t i = 0; i < half; i++) fr.f[i] = powf(10000.0f, -(float)i / (float)half);
    trig_fill_kernel<<<dim3((unsigned)((need_trig + 255) / 256)), dim3(256), 0, c->stream>>>(sc->trig, fr, backlog, half);
    HIP_TRY(hipGetLastError());
    LV_TRY(zero_async(sc->counters, sizeof sc->counters, c->stream));
    return launch_attention(c->stream, out, static_cast<const uint16_t *>(kcache), static_cast<const uint16_t *>(vcache), q, sc->trig,
                            sc->part, sc->counters, nullptr, pos, backlog, heads, rot, batch);
}

// -----------------------------------------------------------------------------------------------------------
// model
// -----------------------------------------------------------------------------------------------------------
static const lv_tensor_desc *find_desc(const lv_tensor_desc *t, uint32_t n, const std::string &name)
{
    for (uint32_t i = 0; i < n; i++)
        if (t[i].name && name == t[i].name) return &t[i];
    const std::string alt = name + ".weight";  // same fallback as ggml_file::get_buffer_descriptor
    for (uint32_t i = 0; i < n; i++)
        if (t[i].name && alt == t[i].name) return &t[i];
    return nullptr;
}

// Persistent-kernel form of the weights: a second copy laid out as per-wave tile streams (lv_mega.h).
// Built when the model has a compiled shape class and all matrices have one type and one kind of scale plane.
template <class S>
static int build_mega_stream(lv_model *m)
{
    lv_ctx *c = m->ctx;
    const uint32_t L = m->hp.layers, D = m->hp.dim;
    const size_t total = (size_t)L * S::LAYER_BYTES + S::HEAD_BYTES + S::TILE;  // + the all-zero dummy tile
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&m->mega_stream), total);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&m->mega_norms), ((size_t)L * 2 + 1) * D * 4);
    if (e != hipSuccess)
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "persistent weight stream of %llu bytes: %s",
                    (unsigned long long)total, hipGetErrorString(e));
    auto pack = [&](uint8_t *dst, int phase, int tiles, const MatView &a, const MatView &b, const MatView &cc) -> int {
        MegaPackSrc src{};
        src.m[0] = a; src.m[1] = b; src.m[2] = cc;
        const size_t threads = (size_t)kMegaWGs * S::NW * tiles * 64;
        mega_pack_kernel<S><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, c->stream>>>(dst, src, phase, m->hp.vocab);
        HIP_TRY(hipGetLastError());
        return LV_OK;
    };
    const MatView none{};
    LV_TRY(zero_async(m->mega_stream + (size_t)L * S::LAYER_BYTES + S::HEAD_BYTES, S::TILE, c->stream));
    for (uint32_t i = 0; i < L; i++) {
        const LayerWeights &lw = m->layers[i];
        uint8_t *base = m->mega_stream + (size_t)i * S::LAYER_BYTES;
        LV_TRY(pack(base, 0, S::TA, lw.wq.view, lw.wk.view, lw.wv.view));
        LV_TRY(pack(base + S::PHASE_A_BYTES, 1, S::TC, lw.wo.view, none, none));
        LV_TRY(pack(base + S::PHASE_A_BYTES + S::PHASE_C_BYTES, 2, S::TD, lw.w3.view, lw.w1.view, none));
        LV_TRY(pack(base + S::PHASE_A_BYTES + S::PHASE_C_BYTES + S::PHASE_D_BYTES, 3, S::TE, lw.w2.view, none, none));
        HIP_TRY(hipMemcpyAsync(m->mega_norms + (size_t)i * 2 * D, lw.attn_norm, (size_t)D * 4, hipMemcpyDeviceToDevice, c->stream));
        HIP_TRY(hipMemcpyAsync(m->mega_norms + ((size_t)i * 2 + 1) * D, lw.ffn_norm, (size_t)D * 4, hipMemcpyDeviceToDevice, c->stream));
    }
    LV_TRY(pack(m->mega_stream + (size_t)L * S::LAYER_BYTES, 4, S::HEAD, m->output.view, none, none));
    HIP_TRY(hipMemcpyAsync(m->mega_norms + (size_t)L * 2 * D, m->norm, (size_t)D * 4, hipMemcpyDeviceToDevice, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return LV_OK;
}

static int build_mega(lv_model *m)
{
    const lv_hparams &hp = m->hp;
    const uint32_t ft = m->output.ftype;
    // one weight type and one kind of scale plane (fp16, or the fp32 one of a version-1 file) throughout
    const bool sf32 = m->output.view.scales_f32 != nullptr;
    bool uniform = ft == LV_Q4_0 || ft == LV_Q8_0;
    for (const LayerWeights &lw : m->layers)
        for (const lv_matrix *x : {&lw.wq, &lw.wk, &lw.wv, &lw.wo, &lw.w1, &lw.w2, &lw.w3})
            uniform = uniform && x->ftype == ft && (x->view.scales_f32 != nullptr) == sf32;
    if (!uniform || (int)m->ctx->props.multiProcessorCount < kMegaWGs) return LV_OK;
    for (int kind = 1; kind <= kMegaKinds; kind++) {
        bool fits = false;
        (void)mega_dispatch(kind, [&](auto shape) -> int {
            using S = decltype(shape);
            fits = hp.dim == (uint32_t)S::D && hp.ff == (uint32_t)S::F && hp.heads == (uint32_t)S::H && ft == (S::QT == 4 ? LV_Q4_0 : LV_Q8_0) && S::SF32 == sf32 &&
                   (hp.vocab + kMegaWGs - 1) / kMegaWGs <= (uint32_t)S::MAX_VOCAB_ROWS;
            return LV_OK;
        });
        if (!fits) continue;
        LV_TRY(mega_dispatch(kind, [&](auto shape) { return build_mega_stream<decltype(shape)>(m); }));
        if (m->tok_ftype != LV_F32) {
            // llava_buffer.cpp:339-401 dequantises the token's row on the host at every step; here the whole table is
            // expanded once (exact: a code times an fp16 scale is representable in fp32)
            const uint64_t nb = (uint64_t)hp.vocab * (hp.dim / 32);
            hipError_t e = hipMalloc(reinterpret_cast<void **>(&m->tok_f32_own), nb * 32 * sizeof(float));
            if (e != hipSuccess)
                return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "fp32 embedding table of %llu bytes: %s",
                            (unsigned long long)(nb * 128), hipGetErrorString(e));
            const unsigned grid = (unsigned)((nb + 255) / 256);
            if (m->tok_ftype == LV_Q4_0) dequant_kernel<4><<<dim3(grid), dim3(256), 0, m->ctx->stream>>>(m->tok_quant.view, 0, nb, m->tok_f32_own);
            else dequant_kernel<8><<<dim3(grid), dim3(256), 0, m->ctx->stream>>>(m->tok_quant.view, 0, nb, m->tok_f32_own);
            HIP_TRY(hipGetLastError());
            HIP_TRY(hipStreamSynchronize(m->ctx->stream));
            m->tok_f32 = m->tok_f32_own;
        }
        m->mega_kind = kind;
        break;
    }
    return LV_OK;
}

struct Want {
    std::string name;
    uint32_t rows, cols;   // expected shape (cols == 1 for vectors)
    bool quant;            // must be q4_0 / q8_0 (matrices); otherwise f32 (vectors) or anything (embeddings)
    const lv_tensor_desc *desc = nullptr;
    uint64_t arena_off = 0;
};

extern "C" int lv_model_upload(lv_ctx *c, const void *base, uint64_t base_size, const lv_hparams *hp,
                               const lv_tensor_desc *table, uint32_t n_tensors, lv_model **out)
{
    if (!c || !base || !hp || !table || !out) return fail(LV_ERR_ARG, "lv_model_upload: null argument");
    *out = nullptr;
    const uint32_t D = hp->dim, F = hp->ff, V = hp->vocab, L = hp->layers;
    if (!D || !F || !V || !L || !hp->heads || hp->heads * hp->rot != D || D % 32 || F % 32)
        return fail(LV_ERR_ARG, "lv_model_upload: inconsistent hyper-parameters (dim %u heads %u rot %u ff %u)", D, hp->heads, hp->rot, F);
    if (hp->rot != 32 && hp->rot != 64 && hp->rot != 128)
        return fail(LV_ERR_ARG, "lv_model_upload: head size %u (32, 64 and 128 are built)", hp->rot);
    HIP_TRY(hipSetDevice(c->device));

    // the tensors the decode path reads, in arena order
    std::vector<Want> wants;
    wants.push_back({"tok_embeddings", V, D, false});
    wants.push_back({"norm", D, 1, false});
    wants.push_back({"output", V, D, true});
    static const char *mats[7] = {"attention.wq", "attention.wk", "attention.wv", "attention.wo",
                                  "feed_forward.w1", "feed_forward.w2", "feed_forward.w3"};
    for (uint32_t i = 0; i < L; i++) {
        const std::string p = "layers." + std::to_string(i) + ".";
        for (int k = 0; k < 7; k++) {
            uint32_t rows = D, cols = D;
            if (k == 4 || k == 6) rows = F;
            if (k == 5) cols = F;
            wants.push_back({p + mats[k], rows, cols, true});
        }
        wants.push_back({p + "attention_norm", D, 1, false});
        wants.push_back({p + "ffn_norm", D, 1, false});
    }

    uint64_t arena_bytes = 0, staging_bytes = 0;
    for (Want &w : wants) {
        w.desc = find_desc(table, n_tensors, w.name);
        if (!w.desc) return fail(LV_ERR_MISSING, "lv_model_upload: tensor %s is not in the table", w.name.c_str());
        const lv_tensor_desc &d = *w.desc;
        if (d.rows != w.rows || d.cols != w.cols)
            return fail(LV_ERR_ARG, "lv_model_upload: %s is %u x %u, expected %u x %u", d.name, d.rows, d.cols, w.rows, w.cols);
        const uint64_t raw = ggml_bytes(d.ftype, (uint64_t)d.rows * d.cols, hp->file_version);
        if (raw == 0 || d.size != raw || d.offset + raw > base_size)
            return fail(LV_ERR_ARG, "lv_model_upload: %s has type %u / %llu bytes at %llu (file holds %llu)", d.name, d.ftype,
                        (unsigned long long)d.size, (unsigned long long)d.offset, (unsigned long long)base_size);
        const bool is_quant = d.ftype == LV_Q4_0 || d.ftype == LV_Q8_0;
        if (w.quant || (is_quant && w.cols > 1)) {
            LV_TRY(check_quant_shape(d.name, d.ftype, hp->file_version, d.rows, d.cols));
            w.arena_off = arena_bytes;
            arena_bytes += matrix_device_bytes(d.ftype, d.rows, d.cols, hp->file_version);
            if (raw > staging_bytes) staging_bytes = raw;
        } else {
            if (d.ftype != LV_F32) return fail(LV_ERR_ARG, "lv_model_upload: %s must be f32 (type %u)", d.name, d.ftype);
            w.arena_off = arena_bytes;
            arena_bytes += align_up(raw, 256);
        }
    }

    lv_model *m = new (std::nothrow) lv_model;
    if (!m) return fail(LV_ERR_OOM, "lv_model_upload: host allocation");
    m->ctx = c;
    m->hp = *hp;
    m->layers.resize(L);
    uint8_t *staging = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&m->arena), arena_bytes);
    if (e == hipSuccess && staging_bytes) e = hipMalloc(reinterpret_cast<void **>(&staging), staging_bytes);
    if (e != hipSuccess) {
        (void)hipFree(m->arena);
        delete m;
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "lv_model_upload: arena of %llu bytes: %s",
                    (unsigned long long)arena_bytes, hipGetErrorString(e));
    }
    m->arena_bytes = arena_bytes;

    int rc = LV_OK;
    const uint8_t *hb = static_cast<const uint8_t *>(base);
    auto put_matrix = [&](const Want &w, lv_matrix *dst) {
        return place_matrix(c, dst, m->arena + w.arena_off, hb + w.desc->offset, w.desc->ftype, w.desc->rows, w.desc->cols, staging, hp->file_version);
    };
    auto put_f32 = [&](const Want &w, const float **dst) -> int {
        HIP_TRY(hipMemcpyAsync(m->arena + w.arena_off, hb + w.desc->offset, w.desc->size, hipMemcpyHostToDevice, c->stream));
        HIP_TRY(hipStreamSynchronize(c->stream));
        *dst = reinterpret_cast<const float *>(m->arena + w.arena_off);
        return LV_OK;
    };
    size_t wi = 0;
    {
        const Want &tok = wants[wi++];
        m->tok_ftype = tok.desc->ftype;
        if (m->tok_ftype == LV_F32) rc = put_f32(tok, &m->tok_f32);
        else rc = put_matrix(tok, &m->tok_quant);
    }
    if (rc == LV_OK) rc = put_f32(wants[wi++], &m->norm);
    if (rc == LV_OK) rc = put_matrix(wants[wi++], &m->output);
    for (uint32_t i = 0; i < L && rc == LV_OK; i++) {
        LayerWeights &lw = m->layers[i];
        lv_matrix *dsts[7] = {&lw.wq, &lw.wk, &lw.wv, &lw.wo, &lw.w1, &lw.w2, &lw.w3};
        for (int k = 0; k < 7 && rc == LV_OK; k++) rc = put_matrix(wants[wi++], dsts[k]);
        if (rc == LV_OK) rc = put_f32(wants[wi++], &lw.attn_norm);
        if (rc == LV_OK) rc = put_f32(wants[wi++], &lw.ffn_norm);
        if (rc == LV_OK && (lw.w1.ftype != lw.w3.ftype)) rc = fail(LV_ERR_ARG, "lv_model_upload: layer %u w1/w3 types differ", i);
    }
    (void)hipFree(staging);
    if (rc == LV_OK) rc = build_mega(m);
    if (rc != LV_OK) {
        (void)hipFree(m->mega_stream);
        (void)hipFree(m->mega_norms);
        (void)hipFree(m->tok_f32_own);
        (void)hipFree(m->arena);
        delete m;
        return rc;
    }
    *out = m;
    return LV_OK;
}

extern "C" int lv_model_destroy(lv_model *m)
{
    if (!m) return LV_OK;
    (void)hipSetDevice(m->ctx->device);
    (void)hipFree(m->prompt_arena);
    (void)hipFree(m->output_copy);
    (void)hipFree(m->mega_stream);
    (void)hipFree(m->mega_norms);
    (void)hipFree(m->tok_f32_own);
    (void)hipFree(m->arena);
    delete m;
    return LV_OK;
}

extern "C" int lv_model_hparams(const lv_model *m, lv_hparams *out)
{
    if (!m || !out) return fail(LV_ERR_ARG, "lv_model_hparams: null argument");
    *out = m->hp;
    return LV_OK;
}

extern "C" int lv_model_arena_bytes(const lv_model *m, uint64_t *bytes)
{
    if (!m || !bytes) return fail(LV_ERR_ARG, "lv_model_arena_bytes: null argument");
    *bytes = m->arena_bytes;
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// session
// -----------------------------------------------------------------------------------------------------------
static void drop_graph(lv_session *s)
{
    if (s->graph_exec) (void)hipGraphExecDestroy(s->graph_exec);
    if (s->graph) (void)hipGraphDestroy(s->graph);
    s->graph_exec = nullptr;
    s->graph = nullptr;
}

extern "C" int lv_session_destroy(lv_session *s)
{
    if (!s) return LV_OK;
    (void)hipSetDevice(s->model->ctx->device);
    if (s->stream) (void)hipStreamSynchronize(s->stream);
    {
        std::lock_guard<std::mutex> lock(s->model->ctx->mega_mutex);
        if (s->model->ctx->mega_last == s) s->model->ctx->mega_last = nullptr;   // its last launch has finished (stream synchronised)
    }
    drop_graph(s);
    void *dev[] = {s->kv, s->trig, s->trig_abs, s->x, s->xn, s->q, s->k, s->v, s->vo, s->ff, s->logits, s->attn_part, s->attn_counters,
                   s->cfg, s->argmax_dev, s->trace_buf, s->trace_attn, s->pf_x, s->pf_xn, s->pf_q, s->pf_k, s->pf_v, s->pf_vo, s->pf_g1, s->pf_g2,
                   s->pf_xh, s->pf_xl, s->pf_xs, s->pf_planes, s->pf_fh, s->pf_fl, s->logits_all};
    for (void *p : dev) (void)hipFree(p);
    for (int i = 0; i < 2; i++) {
        uncached_give(s->model->ctx->device, s->xchg[i], s->xchg_bytes, s->xchg_pooled[i]);
        (void)hipFree(s->xl[i]);
    }
    if (s->status_host) (void)hipHostFree(s->status_host);
    if (s->cfg_host) (void)hipHostFree(s->cfg_host);
    if (s->argmax_host) (void)hipHostFree(s->argmax_host);
    if (s->ev_start) (void)hipEventDestroy(s->ev_start);
    if (s->ev_stop) (void)hipEventDestroy(s->ev_stop);
    if (s->stream) (void)hipStreamDestroy(s->stream);
    delete s;
    return LV_OK;
}

static int session_alloc(lv_session *s)
{
    const lv_hparams &hp = s->model->hp;
    const size_t D = hp.dim, F = hp.ff, V = hp.vocab;
    HIP_TRY(hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->x), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->xn), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->q), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->k), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->v), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->vo), D * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->ff), F * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->logits), V * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->cfg), (1 + kMaxStepTokens) * 4));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->argmax_dev), 4));
    HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->cfg_host), (1 + kMaxStepTokens) * 4, hipHostMallocDefault));
    HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->argmax_host), 4, hipHostMallocDefault));
    if (s->model->mega_kind) {
        size_t bytes = 0, local_bytes = 0;
        LV_TRY(mega_dispatch(s->model->mega_kind, [&](auto shape) -> int {
            bytes = ((size_t)hp.layers * decltype(shape)::XCHG_LAYER + decltype(shape)::XCHG_TAIL) * 4;
            local_bytes = (size_t)hp.layers * decltype(shape)::LOCAL_LAYER * 4;
            return LV_OK;
        }));
        s->xchg_bytes = bytes;
        for (int i = 0; i < 2; i++) {
            LV_TRY(uncached_take(s->model->ctx->device, reinterpret_cast<void **>(&s->xchg[i]), bytes, &s->xchg_pooled[i]));
            HIP_TRY(hipMemsetAsync(s->xchg[i], 0xff, bytes, s->stream));
            HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->xl[i]), local_bytes));
            HIP_TRY(hipMemsetAsync(s->xl[i], 0xff, local_bytes, s->stream));
        }
        HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->status_host), 4096, hipHostMallocDefault));
        memset(s->status_host, 0, 4096);
        HIP_TRY(hipStreamSynchronize(s->stream));
    }
    return LV_OK;
}

extern "C" int lv_session_create(lv_model *m, lv_session **out)
{
    if (!m || !out) return fail(LV_ERR_ARG, "lv_session_create: null argument");
    *out = nullptr;
    HIP_TRY(hipSetDevice(m->ctx->device));
    lv_session *s = new (std::nothrow) lv_session;
    if (!s) return fail(LV_ERR_OOM, "lv_session_create: host allocation");
    s->model = m;
    int rc = session_alloc(s);
    if (rc != LV_OK) {
        lv_session_destroy(s);
        return rc;
    }
    *out = s;
    return LV_OK;
}

// record mode's attention weights: one [backlog][heads] buffer per layer and row of a step, zero until a traced step fills it
static int make_trace_attn(lv_session *s, uint32_t backlog)
{
    const lv_hparams &hp = s->model->hp;
    const size_t bytes = (size_t)hp.layers * s->trace_cap * backlog * hp.heads * 4;
    if (bytes == 0) return LV_OK;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&s->trace_attn), bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        s->trace_attn = nullptr;
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "record mode: attention weights of %u steps rows x %u cache rows: %s", s->trace_cap, backlog,
                    hipGetErrorString(e));
    }
    return zero_async(s->trace_attn, bytes, s->stream);
}

// room for the trace buffers of a step of `rows` tokens (the reference re-creates its buffers when the batch size
// changes, llava_layer_session_data.cpp:60-61; here they only grow).  What an earlier step left is dropped on growth.
static int trace_reserve(lv_session *s, uint32_t rows)
{
    if (rows <= s->trace_cap) return LV_OK;
    const lv_hparams &hp = s->model->hp;
    const size_t slot = hp.dim > hp.ff ? hp.dim : hp.ff;
    HIP_TRY(hipStreamSynchronize(s->stream));
    (void)hipFree(s->trace_buf);
    (void)hipFree(s->trace_attn);
    s->trace_buf = nullptr;
    s->trace_attn = nullptr;
    s->trace_cap = 0;
    s->trace_n = 0;
    const size_t bytes = (size_t)hp.layers * LV_TRACE_ATTN * rows * slot * 4;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&s->trace_buf), bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        s->trace_buf = nullptr;
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "record mode: buffers for a step of %u rows: %s", rows, hipGetErrorString(e));
    }
    s->trace_cap = rows;
    LV_TRY(zero_async(s->trace_buf, bytes, s->stream));
    return make_trace_attn(s, s->backlog);
}

extern "C" int lv_session_reserve(lv_session *s, uint32_t backlog)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_reserve: session is null");
    if (backlog == 0 || backlog > (1u << 20)) return fail(LV_ERR_RANGE, "lv_session_reserve: backlog %u", backlog);
    if (s->in_flight) return fail(LV_ERR_STATE, "lv_session_reserve: a step is in flight");
    if (backlog == s->backlog) return LV_OK;
    const lv_hparams &hp = s->model->hp;
    HIP_TRY(hipSetDevice(s->model->ctx->device));
    HIP_TRY(hipStreamSynchronize(s->stream));
    drop_graph(s);

    const size_t D = hp.dim, plane_new = (size_t)backlog * D, plane_old = (size_t)s->backlog * D;
    uint16_t *kv_new = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&kv_new), (size_t)hp.layers * 2 * plane_new * 2);
    if (e != hipSuccess)
        return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "lv_session_reserve: cache of %u rows: %s", backlog, hipGetErrorString(e));
    // keep the first min(old, new) rows of every plane, zero the rest (llava_layer_session_data.cpp:100-112)
    const size_t keep_rows = s->backlog < backlog ? s->backlog : backlog;
    int rc = zero_async(kv_new, (size_t)hp.layers * 2 * plane_new * 2, s->stream);
    for (uint32_t pl = 0; pl < hp.layers * 2 && rc == LV_OK && keep_rows; pl++) {
        hipError_t ce = hipMemcpyAsync(kv_new + pl * plane_new, s->kv + pl * plane_old, keep_rows * D * 2, hipMemcpyDeviceToDevice, s->stream);
        if (ce != hipSuccess) rc = fail(LV_ERR_HIP, "lv_session_reserve: copy: %s", hipGetErrorString(ce));
    }
    if (rc == LV_OK && hipStreamSynchronize(s->stream) != hipSuccess) rc = fail(LV_ERR_HIP, "lv_session_reserve: sync failed");
    if (rc != LV_OK) {
        (void)hipFree(kv_new);
        return rc;
    }
    (void)hipFree(s->kv);
    s->kv = kv_new;

    (void)hipFree(s->trig);
    s->trig = nullptr;
    (void)hipFree(s->trig_abs);
    s->trig_abs = nullptr;
    (void)hipFree(s->attn_part);
    s->attn_part = nullptr;
    (void)hipFree(s->attn_counters);
    s->attn_counters = nullptr;
    (void)hipFree(s->trace_attn);
    s->trace_attn = nullptr;
    s->backlog = 0;
    LV_TRY(upload_trig(&s->trig, backlog, hp.rot, s->stream));
    LV_TRY(upload_trig(&s->trig_abs, backlog, hp.rot, s->stream, true));
    const uint32_t splits = (backlog + kAttnChunk - 1) / kAttnChunk;
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->attn_part), attn_part_floats(1, hp.heads, splits, hp.rot) * sizeof(float)));
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&s->attn_counters), (size_t)hp.heads * 4));
    LV_TRY(zero_async(s->attn_counters, (size_t)hp.heads * 4, s->stream));
    if (s->trace_buf) LV_TRY(make_trace_attn(s, backlog));
    HIP_TRY(hipStreamSynchronize(s->stream));
    s->backlog = backlog;
    return LV_OK;
}

extern "C" int lv_session_backlog(const lv_session *s, uint32_t *backlog)
{
    if (!s || !backlog) return fail(LV_ERR_ARG, "lv_session_backlog: null argument");
    *backlog = s->backlog;
    return LV_OK;
}

extern "C" int lv_session_use_graph(lv_session *s, int enable)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_use_graph: session is null");
    s->use_graph = enable != 0;
    return LV_OK;
}

extern "C" int lv_session_set_path(lv_session *s, int path)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_set_path: session is null");
    if (path < LV_PATH_AUTO || path > LV_PATH_PERSISTENT) return fail(LV_ERR_ARG, "lv_session_set_path: path %d", path);
    if (path == LV_PATH_PERSISTENT && s->model->mega_kind == 0)
        return fail(LV_ERR_ARG, "lv_session_set_path: this model has no persistent-kernel form (shape or types not covered)");
    s->path = path;
    s->mega_off = false;  // an explicit choice gives the persistent kernel another try
    s->mega_failures = 0;
    return LV_OK;
}

extern "C" int lv_session_path(const lv_session *s, int *path)
{
    if (!s || !path) return fail(LV_ERR_ARG, "lv_session_path: null argument");
    const int fallback = s->use_graph ? LV_PATH_GRAPH : LV_PATH_KERNELS;
    if (s->path != LV_PATH_AUTO)
        *path = s->path == LV_PATH_PERSISTENT && s->mega_off ? fallback : s->path;
    else
        *path = s->model->mega_kind && !s->mega_off ? LV_PATH_PERSISTENT : fallback;
    return LV_OK;
}

// One token through the persistent kernel.  Its workgroups hand vectors to each other, so all 256 of them have to be
// resident at once: one per CU, on a device of at least 256 CUs that grants the kernel a workgroup per CU (lv_ctx::mega_fits
// asks the runtime once per shape class).  *refused is set, and LV_OK returned, when that does not hold or the launch is
// turned down for lack of resources; nothing has run then.  The launch is an ordinary one: hipLaunchCooperativeKernel's own
// test is the same occupancy arithmetic and adds nothing to it (kernels of other streams can hold CUs for a while under
// either; the waits inside the kernel are bounded for that), the two launch at the same rate (measured in alternation), and
// the separate queue the runtime opens for cooperative launches makes a process under rocprofv3 end with a segmentation
// fault in its exit handlers (a forty-line program with one cooperative launch of an empty kernel does the same).
static int launch_mega(lv_session *s, uint32_t pos, uint32_t token, bool *refused, float *logits_dst)
{
    const lv_model *m = s->model;
    MegaArgs a{};
    a.wstream = m->mega_stream;
    a.norms = m->mega_norms;
    a.tok_f32 = m->tok_f32;
    a.kv = s->kv;
    a.trig = s->trig;
    a.xchg = s->xchg[s->xchg_turn & 1];
    a.xchg_rearm = s->xchg[(s->xchg_turn + 1) & 1];
    a.xl = s->xl[s->xchg_turn & 1];
    a.xl_rearm = s->xl[(s->xchg_turn + 1) & 1];
    a.logits = logits_dst;
    a.status = s->status_host;
    a.layers = m->hp.layers; a.vocab = m->hp.vocab; a.backlog = s->backlog; a.pos = pos; a.token = token;
    a.spin_limit = s->wait_limit ? s->wait_limit : kSpinLimit;
    a.xcd_local = s->xcd_handover ? 1u : 0u;
    s->xchg_turn++;
    void *params[] = {&a};
    lv_ctx *c = m->ctx;
    std::lock_guard<std::mutex> lock(c->mega_mutex);
    if (c->mega_last && c->mega_last != s) HIP_TRY(hipStreamWaitEvent(s->stream, c->mega_done, 0));
    LV_TRY(mega_dispatch(m->mega_kind, [&](auto shape) -> int {
        using S = decltype(shape);
        const void *kernel = reinterpret_cast<const void *>(&mega_decode_kernel<S>);
        int &fits = c->mega_fits[m->mega_kind];
        if (fits < 0) {
            int per_cu = 0;
            const hipError_t oe = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, S::NW * 64, 0);
            if (oe != hipSuccess) (void)hipGetLastError();
            fits = oe == hipSuccess && per_cu >= 1 && c->props.multiProcessorCount >= kMegaWGs ? 1 : 0;
        }
        if (!fits) {
            *refused = true;
            return LV_OK;
        }
        const hipError_t e = hipLaunchKernel(kernel, dim3(kMegaWGs), dim3(S::NW * 64), params, 0, s->stream);
        if (e == hipErrorLaunchOutOfResources || e == hipErrorNotSupported) {
            (void)hipGetLastError();
            *refused = true;
            return LV_OK;
        }
        HIP_TRY(e);
        return LV_OK;
    }));
    if (*refused) {
        s->xchg_turn--;
        return LV_OK;
    }
    if (!c->mega_done) HIP_TRY(hipEventCreateWithFlags(&c->mega_done, hipEventDisableTiming));
    HIP_TRY(hipEventRecord(c->mega_done, s->stream));
    c->mega_last = s;
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// the step
// -----------------------------------------------------------------------------------------------------------
static float *trace_slot(const lv_session *s, uint32_t layer, int which, uint32_t row)
{
    const lv_hparams &hp = s->model->hp;
    const size_t slot = hp.dim > hp.ff ? hp.dim : hp.ff;
    return s->trace_buf + (((size_t)layer * LV_TRACE_ATTN + which) * s->trace_cap + row) * slot;
}

static float *trace_attn_slot(const lv_session *s, uint32_t layer, uint32_t row)
{
    return s->trace_attn + ((size_t)layer * s->trace_cap + row) * s->backlog * s->model->hp.heads;
}

// row = the token's index in its step
static int trace_copy(lv_session *s, uint32_t layer, int which, uint32_t row, const float *src, size_t count)
{
    if (!s->trace) return LV_OK;
    float *dst = trace_slot(s, layer, which, row);
    HIP_TRY(hipMemcpyAsync(dst, src, count * 4, hipMemcpyDeviceToDevice, s->stream));
    return LV_OK;
}

// One token through every layer (llava_layer.cpp:53-73 + llava_command_buffer.cpp:38-39).  The token id is
// cfg[1 + idx], its cache row cfg[0] + idx.  With_head = also compute the logits.
static int record_token(lv_session *s, uint32_t idx, bool with_head)
{
    const lv_model *m = s->model;
    const lv_hparams &hp = m->hp;
    const uint32_t D = hp.dim, F = hp.ff;
    hipStream_t st = s->stream;
    const uint32_t *pos_ptr = s->cfg, *tok_ptr = s->cfg + 1 + idx;

    if (m->tok_ftype == LV_F32)
        embed_f32_kernel<<<dim3((D + 255) / 256, 1), dim3(256), 0, st>>>(s->x, m->tok_f32, tok_ptr, D);
    else if (m->tok_ftype == LV_Q4_0)
        embed_quant_kernel<4><<<dim3((D / 32 + 63) / 64, 1), dim3(64), 0, st>>>(s->x, m->tok_quant.view, tok_ptr);
    else
        embed_quant_kernel<8><<<dim3((D / 32 + 63) / 64, 1), dim3(64), 0, st>>>(s->x, m->tok_quant.view, tok_ptr);
    HIP_TRY(hipGetLastError());

    const dim3 kv_grid((D + 255) / 256, 1);
    for (uint32_t li = 0; li < hp.layers; li++) {
        const LayerWeights &lw = m->layers[li];
        float *const outs[3] = {s->k, s->q, s->v};
        const lv_matrix *const mats[3] = {&lw.wk, &lw.wq, &lw.wv};
        // Without tracing, at shapes the streaming kernel covers, normalisation and the cache append ride along with
        // the projections (one launch instead of five); the trace wants the normalised vector in memory.
        const bool fused = !s->trace && gemv3_streams(mats) && gemv_streams(lw.w3.view, 1);
        if (fused) {
            Gemv3Extras ex;
            ex.norm_w = lw.attn_norm;
            ex.cache[0] = kv_ptr(s, li, 0); ex.cache[2] = kv_ptr(s, li, 1);
            ex.pos_ptr = pos_ptr; ex.pos_add = idx; ex.backlog = s->backlog;
            LV_TRY(launch_gemv3(st, outs, mats, s->x, &ex));
        } else {
            normalize_kernel<<<dim3(1), dim3(256), 0, st>>>(s->xn, s->x, lw.attn_norm, D);
            HIP_TRY(hipGetLastError());
            LV_TRY(trace_copy(s, li, LV_TRACE_NORM_IN, idx, s->xn, D));
            LV_TRY(launch_gemv3(st, outs, mats, s->xn));
            kv_append2_kernel<<<dim3(kv_grid.x, kv_grid.y, 2), dim3(256), 0, st>>>(kv_ptr(s, li, 0), kv_ptr(s, li, 1), s->k, s->v, pos_ptr, idx, D, s->backlog);
            HIP_TRY(hipGetLastError());
        }
        LV_TRY(launch_attention(st, s->vo, kv_ptr(s, li, 0), kv_ptr(s, li, 1), s->q, s->trig, s->attn_part, s->attn_counters,
                                pos_ptr, idx, s->backlog, hp.heads, hp.rot, 1));
        if (s->trace) {
            attn_weights_kernel<<<dim3(hp.heads), dim3(256), 0, st>>>(trace_attn_slot(s, li, idx), kv_ptr(s, li, 0), s->q,
                                                                       s->trig, pos_ptr, idx, hp.heads, hp.rot, s->backlog);
            HIP_TRY(hipGetLastError());
        }
        LV_TRY(launch_gemv(st, s->x, lw.wo, nullptr, s->vo, 1, kGemvAdd));
        LV_TRY(trace_copy(s, li, LV_TRACE_POST_ATTN, idx, s->x, D));
        if (fused) {
            LV_TRY(launch_gemv(st, s->ff, lw.w3, &lw.w1, s->x, 1, kGemvSilu, lw.ffn_norm));
        } else {
            normalize_kernel<<<dim3(1), dim3(256), 0, st>>>(s->xn, s->x, lw.ffn_norm, D);
            HIP_TRY(hipGetLastError());
            LV_TRY(trace_copy(s, li, LV_TRACE_POST_ATTN_NORM, idx, s->xn, D));
            LV_TRY(launch_gemv(st, s->ff, lw.w3, &lw.w1, s->xn, 1, kGemvSilu));
        }
        LV_TRY(trace_copy(s, li, LV_TRACE_FF, idx, s->ff, F));
        LV_TRY(launch_gemv(st, s->x, lw.w2, nullptr, s->ff, 1, kGemvAdd));
        LV_TRY(trace_copy(s, li, LV_TRACE_OUT, idx, s->x, D));
    }
    if (with_head) {
        if (!s->trace && gemv_streams(m->output.view, 1)) {
            LV_TRY(launch_gemv(st, s->logits, m->output, nullptr, s->x, 1, kGemvStore, m->norm));
        } else {
            normalize_kernel<<<dim3(1), dim3(256), 0, st>>>(s->xn, s->x, m->norm, D);
            HIP_TRY(hipGetLastError());
            LV_TRY(launch_gemv(st, s->logits, m->output, nullptr, s->xn, 1, kGemvStore));
        }
    }
    return LV_OK;
}

// ---- batched prompt evaluation -----------------------------------------------------------------------------
// The prompt copy of every layer matrix, made when a model evaluates its first batch (2 bytes a weight: 13.5 GB for a
// 7B model; decode never reads it).  False when the device has no room for it: batches then go token by token.
static bool ensure_prompt_copy(lv_model *m)
{
    std::lock_guard<std::mutex> lock(m->prompt_mutex);
    if (m->prompt_state) return m->prompt_state > 0;
    uint64_t halfs = 0;
    for (LayerWeights &lw : m->layers) {
        const bool pair = gemm_pairable(lw.w3, lw.w1);
        for (lv_matrix *x : {&lw.wq, &lw.wk, &lw.wv, &lw.wo, &lw.w2}) halfs += prompt_copy_halfs(*x);
        halfs += pair ? pair_copy_halfs(lw.w3) : prompt_copy_halfs(lw.w1) + prompt_copy_halfs(lw.w3);
    }
    m->prompt_state = -1;
    if (hipMalloc(reinterpret_cast<void **>(&m->prompt_arena), halfs * 2) != hipSuccess) {
        (void)hipGetLastError();
        m->prompt_arena = nullptr;
        return false;
    }
    uint16_t *at = m->prompt_arena;
    hipStream_t st = m->ctx->stream;
    for (LayerWeights &lw : m->layers) {
        const bool pair = gemm_pairable(lw.w3, lw.w1);
        for (lv_matrix *x : {&lw.wq, &lw.wk, &lw.wv, &lw.wo, &lw.w2, &lw.w1, &lw.w3}) {
            if (pair && (x == &lw.w1 || x == &lw.w3)) continue;
            if (launch_expand(st, at, *x) != LV_OK) return false;
            x->h16 = at;
            at += prompt_copy_halfs(*x);
        }
        if (pair) {
            if (launch_expand_pair(st, at, lw.w3, lw.w1) != LV_OK) return false;
            lw.gate_up16 = at;
            at += pair_copy_halfs(lw.w3);
        }
    }
    if (hipStreamSynchronize(st) != hipSuccess) return false;
    m->prompt_state = 1;
    return true;
}

// the prompt copy of the output matrix: only a batch that keeps the logits of every row multiplies all its rows by it
static bool ensure_output_copy(lv_model *m)
{
    std::lock_guard<std::mutex> lock(m->prompt_mutex);
    if (m->output_state) return m->output_state > 0;
    m->output_state = -1;
    if (m->output.view.cols % 32 || (m->output.ftype != LV_Q4_0 && m->output.ftype != LV_Q8_0)) return false;
    if (hipMalloc(reinterpret_cast<void **>(&m->output_copy), (size_t)prompt_copy_halfs(m->output) * 2) != hipSuccess) {
        (void)hipGetLastError();
        m->output_copy = nullptr;
        return false;
    }
    if (launch_expand(m->ctx->stream, m->output_copy, m->output) != LV_OK || hipStreamSynchronize(m->ctx->stream) != hipSuccess) return false;
    m->output.h16 = m->output_copy;
    m->output_state = 1;
    return true;
}

constexpr uint32_t kPrefillChunk = 512;    // tokens evaluated together (bounds the workspace)

static int prefill_reserve(lv_session *s, uint32_t n)
{
    const lv_hparams &hp = s->model->hp;
    const size_t D = hp.dim, F = hp.ff;
    const uint32_t cap = (n + kGemmTile - 1) / kGemmTile * kGemmTile;
    if (cap > s->pf_cap) {
        HIP_TRY(hipStreamSynchronize(s->stream));
        void **bufs[] = {(void **)&s->pf_x, (void **)&s->pf_xn, (void **)&s->pf_q, (void **)&s->pf_k, (void **)&s->pf_v, (void **)&s->pf_vo,
                         (void **)&s->pf_g1, (void **)&s->pf_g2, (void **)&s->pf_xh, (void **)&s->pf_xl, (void **)&s->pf_xs,
                         (void **)&s->pf_fh, (void **)&s->pf_fl};
        const size_t halfs = gemm_k_padded((uint32_t)(F > D ? F : D)) * 2;   // an activation half: padded K, 2 bytes each
        const size_t sizes[] = {D * 4, D * 4, D * 4, D * 4, D * 4, D * 4, F * 4, F * 4, halfs, halfs, 4, halfs, halfs};
        s->pf_cap = 0;
        for (int i = 0; i < 13; i++) {
            (void)hipFree(*bufs[i]);
            *bufs[i] = nullptr;
            hipError_t e = hipMalloc(bufs[i], sizes[i] * cap);
            if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "prompt workspace: %s", hipGetErrorString(e));
        }
        s->pf_cap = cap;
    }
    const size_t planes = 4 * attn_plane_halfs(s->backlog, hp.heads, hp.rot);
    if (planes > s->pf_plane_halfs) {
        HIP_TRY(hipStreamSynchronize(s->stream));
        (void)hipFree(s->pf_planes);
        s->pf_planes = nullptr;
        s->pf_plane_halfs = 0;
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&s->pf_planes), planes * 2);
        if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "prompt workspace: %s", hipGetErrorString(e));
        s->pf_plane_halfs = planes;
    }
    return LV_OK;
}

// x += pending K slices, xn = normalize(x) * w, halves of xn for the next GEMM: one kernel where the
// row fits its registers, else the three separate ones.  xn (fp32) is written only when want_xn.  *xscale: the per-token
// scale the GEMMs that read these halves have to apply (null when the halves are unscaled).
static int launch_prefill_norm(hipStream_t st, lv_session *s, const float *w, uint32_t n, uint32_t D, float *const parts[kGemmMaxMats],
                               uint32_t pending, bool want_xn, const float **xscale)
{
    *xscale = nullptr;
    const uint32_t n_pad = (n + kGemmTile - 1) / kGemmTile * kGemmTile;
    if (D <= 8192 && D % 8 == 0) {
        PrefillNormArgs a{};
        a.x = s->pf_x; a.nparts = pending; a.w = w; a.xn = want_xn ? s->pf_xn : nullptr; a.xh = s->pf_xh; a.xl = s->pf_xl; a.dim = D; a.n = n;
        a.Kp = gemm_k_padded(D);
        a.xscale = s->pf_xs;
        for (uint32_t i = 0; i < pending; i++) a.parts[i] = parts[i];
        prefill_norm_kernel<<<dim3(n_pad), dim3(256), 0, st>>>(a);
        HIP_TRY(hipGetLastError());
        *xscale = s->pf_xs;
        return LV_OK;
    }
    if (pending) LV_TRY(launch_gemm_reduce(st, s->pf_x, D, parts, pending, D, n, true));
    normalize_kernel<<<dim3(n), dim3(256), 0, st>>>(s->pf_xn, s->pf_x, w, D);
    HIP_TRY(hipGetLastError());
    *xscale = s->pf_xs;
    return launch_split(st, s->pf_xh, s->pf_xl, s->pf_xs, s->pf_xn, n, D);
}

// Rows idx0 .. idx0+n-1 of the step at once (llava_layer.cpp:39-75 with batch > 1).  Row z sees cache rows
// 0..pos+z: all K/V rows of the chunk are appended before any row attends, rows above its own are masked.
static int record_prefill(lv_session *s, uint32_t idx0, uint32_t n, bool with_head, uint32_t row_base)
{
    const lv_model *m = s->model;
    const lv_hparams &hp = m->hp;
    const uint32_t D = hp.dim, F = hp.ff;
    hipStream_t st = s->stream;
    const uint32_t *pos_ptr = s->cfg, *tok_ptr = s->cfg + 1 + idx0;
    LV_TRY(prefill_reserve(s, n));

    if (m->tok_ftype == LV_F32)
        embed_f32_kernel<<<dim3((D + 255) / 256, n), dim3(256), 0, st>>>(s->pf_x, m->tok_f32, tok_ptr, D);
    else if (m->tok_ftype == LV_Q4_0)
        embed_quant_kernel<4><<<dim3((D / 32 + 63) / 64, n), dim3(64), 0, st>>>(s->pf_x, m->tok_quant.view, tok_ptr);
    else
        embed_quant_kernel<8><<<dim3((D / 32 + 63) / 64, n), dim3(64), 0, st>>>(s->pf_x, m->tok_quant.view, tok_ptr);
    HIP_TRY(hipGetLastError());

    // q, k and v buffers of a layer are free once attention has run: they take the K slices of the output projection
    // and of the down projection; `pending` of them wait to be added to the residual stream by the next norm
    float *const parts[kGemmMaxMats] = {s->pf_q, s->pf_k, s->pf_v, s->pf_vo};
    uint32_t pending = 0;
    for (uint32_t li = 0; li < hp.layers; li++) {
        const LayerWeights &lw = m->layers[li];
        const bool qkv_same = gemm_same(lw.wq, lw.wk) && gemm_same(lw.wq, lw.wv), gate_same = gemm_same(lw.w3, lw.w1);
        const float *xscale = nullptr;
        LV_TRY(launch_prefill_norm(st, s, lw.attn_norm, n, D, parts, pending, !qkv_same, &xscale));
        pending = 0;
        const bool kv_in_cache = qkv_same && lw.wq.view.rows == D;     // the GEMM's epilogue is the cache append of the batch
        if (kv_in_cache) {
            LV_TRY(launch_gemm_qkv(st, s->pf_q, kv_ptr(s, li, 0), kv_ptr(s, li, 1), lw.wq, lw.wk, lw.wv, n, s->pf_xh, s->pf_xl, xscale, pos_ptr, idx0,
                                   s->backlog));
        } else if (qkv_same) {
            float *const outs[3] = {s->pf_q, s->pf_k, s->pf_v};
            const lv_matrix *const ws[3] = {&lw.wq, &lw.wk, &lw.wv};
            LV_TRY(launch_gemm_multi(st, outs, D, ws, 3, n, s->pf_xh, s->pf_xl, false, xscale));
        } else {
            LV_TRY(launch_gemm_presplit(st, s->pf_q, D, lw.wq, n, s->pf_xh, s->pf_xl, false, xscale));
            LV_TRY(launch_gemm_presplit(st, s->pf_k, D, lw.wk, n, s->pf_xh, s->pf_xl, false, xscale));
            LV_TRY(launch_gemm_presplit(st, s->pf_v, D, lw.wv, n, s->pf_xh, s->pf_xl, false, xscale));
        }
        // the batch's K and V rows are in the cache already, or go there in the first of the attention kernels
        const float *kin = kv_in_cache ? nullptr : s->pf_k, *vin = kv_in_cache ? nullptr : s->pf_v;
        if (D % kGemmK == 0) {     // the attention kernel writes the halves the output projection reads
            LV_TRY(launch_attention_batch(st, nullptr, s->pf_xh, s->pf_xl, D, s->pf_planes, kv_ptr(s, li, 0), kv_ptr(s, li, 1), kin, vin, s->pf_q, s->trig_abs,
                                          pos_ptr, idx0, n, s->backlog, hp.heads, hp.rot));
        } else {                   // a padded K: the split kernel writes the zero columns as well
            LV_TRY(launch_attention_batch(st, s->pf_vo, nullptr, nullptr, 0, s->pf_planes, kv_ptr(s, li, 0), kv_ptr(s, li, 1), kin, vin, s->pf_q, s->trig_abs,
                                          pos_ptr, idx0, n, s->backlog, hp.heads, hp.rot));
            LV_TRY(launch_split(st, s->pf_xh, s->pf_xl, nullptr, s->pf_vo, n, D));
        }
        LV_TRY(launch_gemm_sliced(st, s->pf_x, D, lw.wo, n, s->pf_xh, s->pf_xl, nullptr, true, parts, &pending));
        LV_TRY(launch_prefill_norm(st, s, lw.ffn_norm, n, D, parts, pending, !gate_same, &xscale));
        pending = 0;
        const uint16_t *fh = s->pf_xh, *fl = s->pf_xl;     // where the down projection finds its activations
        if (lw.gate_up16) {        // SwiGLU in the GEMM's epilogue
            LV_TRY(launch_gemm_silu(st, s->pf_fh, s->pf_fl, lw.gate_up16, F, D, n, s->pf_xh, s->pf_xl, xscale, s->pf_g1, s->pf_g2));
            fh = s->pf_fh; fl = s->pf_fl;
        } else if (gate_same) {
            float *const outs[2] = {s->pf_g1, s->pf_g2};
            const lv_matrix *const ws[2] = {&lw.w3, &lw.w1};
            LV_TRY(launch_gemm_multi(st, outs, F, ws, 2, n, s->pf_xh, s->pf_xl, false, xscale));
        } else {
            LV_TRY(launch_gemm_presplit(st, s->pf_g1, F, lw.w3, n, s->pf_xh, s->pf_xl, false, xscale));
            LV_TRY(launch_gemm_presplit(st, s->pf_g2, F, lw.w1, n, s->pf_xh, s->pf_xl, false, xscale));
        }
        if (!lw.gate_up16) {   // SwiGLU straight into the fp16 halves the down projection reads
            const uint32_t Fp = gemm_k_padded(F);
            const dim3 grid(Fp / 64, (n + kGemmTile - 1) / kGemmTile * kGemmTile / 32);
            if (F % 8) return fail(LV_ERR_ARG, "prompt batch: ff size %u", F);
            silu_split_kernel<<<grid, dim3(256), 0, st>>>(s->pf_xh, s->pf_xl, s->pf_g1, s->pf_g2, n, F, Fp);
            HIP_TRY(hipGetLastError());
        }
        LV_TRY(launch_gemm_sliced(st, s->pf_x, D, lw.w2, n, fh, fl, nullptr, true, parts, &pending));
    }
    if (s->all_logits) {
        // every row's logits, as the reference computes them (llava_command_buffer.cpp:38-39): final norm of all n rows, then the
        // output matrix on the matrix cores where its prompt copy exists, as a batched GEMV otherwise
        float *dst = s->logits_all + (size_t)(row_base + idx0) * hp.vocab;
        if (ensure_output_copy(s->model)) {
            const float *xscale = nullptr;
            LV_TRY(launch_prefill_norm(st, s, m->norm, n, D, parts, pending, false, &xscale));
            LV_TRY(launch_gemm_presplit(st, dst, hp.vocab, m->output, n, s->pf_xh, s->pf_xl, false, xscale));
        } else {
            if (pending) LV_TRY(launch_gemm_reduce(st, s->pf_x, D, parts, pending, D, n, true));
            normalize_kernel<<<dim3(n), dim3(256), 0, st>>>(s->pf_xn, s->pf_x, m->norm, D);
            HIP_TRY(hipGetLastError());
            LV_TRY(launch_gemv(st, dst, m->output, nullptr, s->pf_xn, n, kGemvStore));
        }
        if (with_head) HIP_TRY(hipMemcpyAsync(s->logits, dst + (size_t)(n - 1) * hp.vocab, (size_t)hp.vocab * 4, hipMemcpyDeviceToDevice, st));
        return LV_OK;
    }
    if (pending) LV_TRY(launch_gemm_reduce(st, s->pf_x, D, parts, pending, D, n, true));
    if (with_head) {
        // only the last row's logits are ever read (llava_session.cpp:131-139)
        normalize_kernel<<<dim3(1), dim3(256), 0, st>>>(s->xn, s->pf_x + (size_t)(n - 1) * D, m->norm, D);
        HIP_TRY(hipGetLastError());
        LV_TRY(launch_gemv(st, s->logits, m->output, nullptr, s->xn, 1, kGemvStore));
    }
    return LV_OK;
}

extern "C" int lv_step_begin(lv_session *s, const uint32_t *tokens, uint32_t n, uint32_t pos)
{
    if (!s || !tokens) return fail(LV_ERR_ARG, "lv_step_begin: null argument");
    if (s->in_flight) return fail(LV_ERR_STATE, "lv_step_begin: the previous step has not been waited for");
    if (n == 0) return fail(LV_ERR_ARG, "lv_step_begin: no tokens");
    if (n > kMaxStepTokens) return fail(LV_ERR_RANGE, "lv_step_begin: %u tokens in one step (limit %u)", n, kMaxStepTokens);
    if (s->backlog == 0) return fail(LV_ERR_STATE, "lv_step_begin: lv_session_reserve has not been called");
    if ((uint64_t)pos + n > s->backlog)
        return fail(LV_ERR_RANGE, "lv_step_begin: rows %u..%u exceed the backlog of %u", pos, pos + n - 1, s->backlog);
    for (uint32_t i = 0; i < n; i++)
        if (tokens[i] >= s->model->hp.vocab) return fail(LV_ERR_RANGE, "lv_step_begin: token id %u of a vocabulary of %u", tokens[i], s->model->hp.vocab);
    HIP_TRY(hipSetDevice(s->model->ctx->device));

    s->have_logits = false;
    s->pick_in_status = false;
    s->logits_rows = 0;
    if (s->all_logits) {
        if (n > s->logits_cap) {
            HIP_TRY(hipStreamSynchronize(s->stream));
            (void)hipFree(s->logits_all);
            s->logits_all = nullptr;
            s->logits_cap = 0;
            const hipError_t e = hipMalloc(reinterpret_cast<void **>(&s->logits_all), (size_t)n * s->model->hp.vocab * 4);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                s->logits_all = nullptr;
                return fail(e == hipErrorOutOfMemory ? LV_ERR_OOM : LV_ERR_HIP, "lv_step_begin: logits of %u rows: %s", n, hipGetErrorString(e));
            }
            s->logits_cap = n;
        }
    }
    const uint32_t n_rows = n, V = s->model->hp.vocab;
    uint32_t row_base = 0;          // rows of this step already launched on the persistent kernel when the rest takes another path
    if (s->trace) {
        LV_TRY(trace_reserve(s, n));
        s->trace_n = n;
    }

    int path = LV_PATH_AUTO;
    (void)lv_session_path(s, &path);
    // the persistent kernel also takes the short steps (a few prompt or add_text tokens) below the size at which the
    // batched path pays: one launch per token, each 1.7 x faster than the operator chain's token
    bool persistent = n < kPrefillMin && path == LV_PATH_PERSISTENT && !s->trace;
    s->mega_step = false;
    if (persistent) {
        uint32_t done = 0;
        bool refused = false;
        while (done < n) {
            LV_TRY(launch_mega(s, pos + done, tokens[done], &refused, s->all_logits ? s->logits_all + (size_t)done * V : s->logits));
            if (refused) break;
            done++;
            s->mega_step = true;
            s->in_flight = true;       // from here on an error return leaves kernels on the stream: lv_step_wait has to follow
        }
        if (refused) {
            // the tokens launched so far stay as they are; the rest of this step, and every later one, takes the other path
            s->mega_off = true;
            persistent = false;
            (void)lv_session_path(s, &path);
            tokens += done; n -= done; pos += done;
            row_base = done;
        } else {
            s->pick_in_status = true;  // the kernel leaves the greedy pick (of the last token) in the pinned status block
            if (s->all_logits)         // lv_logits_read takes the last row from where every path leaves it
                HIP_TRY(hipMemcpyAsync(s->logits, s->logits_all + (size_t)(n - 1) * V, (size_t)V * 4, hipMemcpyDeviceToDevice, s->stream));
        }
    }
    if (!persistent) {             // the persistent kernel takes position and token id as launch arguments
        s->cfg_host[0] = pos;
        memcpy(s->cfg_host + 1, tokens, (size_t)n * 4);
        HIP_TRY(hipMemcpyAsync(s->cfg, s->cfg_host, (size_t)(1 + n) * 4, hipMemcpyHostToDevice, s->stream));
    }
    if (persistent) {
        // launched above
    } else if (n == 1 && (path == LV_PATH_GRAPH || (path == LV_PATH_PERSISTENT && s->use_graph)) && !s->trace) {
        if (!s->graph_exec) {
            HIP_TRY(hipStreamBeginCapture(s->stream, hipStreamCaptureModeThreadLocal));
            int rc = record_token(s, 0, true);
            hipGraph_t g = nullptr;
            hipError_t e = hipStreamEndCapture(s->stream, &g);
            if (rc != LV_OK) {
                if (g) (void)hipGraphDestroy(g);
                return rc;
            }
            HIP_TRY(e);
            s->graph = g;
            HIP_TRY(hipGraphInstantiate(&s->graph_exec, s->graph, nullptr, nullptr, 0));
        }
        HIP_TRY(hipGraphLaunch(s->graph_exec, s->stream));
        if (s->all_logits) HIP_TRY(hipMemcpyAsync(s->logits_all + (size_t)row_base * V, s->logits, (size_t)V * 4, hipMemcpyDeviceToDevice, s->stream));
    } else {
        // rows are evaluated one after the other: row z sees cache rows 0..pos+z, which is what the batched
        // shaders compute (every row's K/V is appended before any row attends, and rows above are masked)
        if (n >= kPrefillMin && !s->trace && ensure_prompt_copy(s->model)) {
            for (uint32_t i = 0; i < n; i += kPrefillChunk) {
                const uint32_t m = n - i < kPrefillChunk ? n - i : kPrefillChunk;
                LV_TRY(record_prefill(s, i, m, i + m == n, row_base));
            }
        } else {
            for (uint32_t i = 0; i < n; i++) {
                LV_TRY(record_token(s, i, s->all_logits || i + 1 == n));
                if (s->all_logits)
                    HIP_TRY(hipMemcpyAsync(s->logits_all + (size_t)(row_base + i) * V, s->logits, (size_t)V * 4, hipMemcpyDeviceToDevice, s->stream));
            }
        }
    }
    s->in_flight = true;
    s->have_logits = true;
    if (s->all_logits) s->logits_rows = n_rows;
    return LV_OK;
}

extern "C" int lv_step_wait(lv_session *s)
{
    if (!s) return fail(LV_ERR_ARG, "lv_step_wait: session is null");
    HIP_TRY(hipStreamSynchronize(s->stream));
    s->in_flight = false;
    const bool mega_step = s->mega_step;
    s->mega_step = false;
    if (s->status_host && *s->status_host) {
        *s->status_host = 0;
        if (++s->mega_failures >= 2) {
            s->mega_off = true;
            return fail(LV_ERR_HIP, "persistent decode kernel: a hand-over wait expired in two steps in a row; this session now takes the %s path",
                        s->use_graph ? "graph" : "operator");
        }
        return fail(LV_ERR_HIP, "persistent decode kernel: a hand-over wait expired (workgroups not co-resident?)");
    }
    if (mega_step) s->mega_failures = 0;
    return LV_OK;
}

extern "C" int lv_logits_read(lv_session *s, float *dst)
{
    if (!s || !dst) return fail(LV_ERR_ARG, "lv_logits_read: null argument");
    if (!s->have_logits) return fail(LV_ERR_STATE, "lv_logits_read: no step has produced logits");
    HIP_TRY(hipMemcpyAsync(dst, s->logits, (size_t)s->model->hp.vocab * 4, hipMemcpyDeviceToHost, s->stream));
    return lv_step_wait(s);
}

extern "C" int lv_session_set_all_logits(lv_session *s, int enable)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_set_all_logits: session is null");
    if (s->in_flight) return fail(LV_ERR_STATE, "lv_session_set_all_logits: a step is in flight");
    s->all_logits = enable != 0;
    if (!s->all_logits) s->logits_rows = 0;
    return LV_OK;
}

extern "C" int lv_logits_read_rows(lv_session *s, uint32_t row0, uint32_t n_rows, float *dst)
{
    if (!s || (n_rows && !dst)) return fail(LV_ERR_ARG, "lv_logits_read_rows: null argument");
    if (!s->have_logits || s->logits_rows == 0) return fail(LV_ERR_STATE, "lv_logits_read_rows: no step has kept the logits of all its rows (lv_session_set_all_logits)");
    if (row0 > s->logits_rows || n_rows > s->logits_rows - row0)
        return fail(LV_ERR_RANGE, "lv_logits_read_rows: rows %u..%u of a step of %u", row0, row0 + n_rows, s->logits_rows);
    if (n_rows) {
        const size_t V = s->model->hp.vocab;
        HIP_TRY(hipMemcpyAsync(dst, s->logits_all + (size_t)row0 * V, (size_t)n_rows * V * 4, hipMemcpyDeviceToHost, s->stream));
    }
    return lv_step_wait(s);
}

extern "C" int lv_argmax(lv_session *s, uint32_t *token)
{
    if (!s || !token) return fail(LV_ERR_ARG, "lv_argmax: null argument");
    if (!s->have_logits) return fail(LV_ERR_STATE, "lv_argmax: no step has produced logits");
    if (s->pick_in_status) {
        LV_TRY(lv_step_wait(s));
        *token = s->status_host[kStatusToken];
        return LV_OK;
    }
    argmax_kernel<<<dim3(1), dim3(1024), 0, s->stream>>>(s->logits, s->model->hp.vocab, s->argmax_dev);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpyAsync(s->argmax_host, s->argmax_dev, 4, hipMemcpyDeviceToHost, s->stream));
    LV_TRY(lv_step_wait(s));
    *token = *s->argmax_host;
    return LV_OK;
}

extern "C" int lv_session_set_xcd_handover(lv_session *s, int enable)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_set_xcd_handover: session is null");
    s->xcd_handover = enable != 0;
    return LV_OK;
}

extern "C" int lv_session_xcd_handover(lv_session *s, int *used)
{
    if (!s || !used) return fail(LV_ERR_ARG, "lv_session_xcd_handover: null argument");
    if (s->in_flight) return fail(LV_ERR_STATE, "lv_session_xcd_handover: a step is in flight");
    *used = s->status_host && s->status_host[kStatusXcd] ? 1 : 0;
    return LV_OK;
}

extern "C" int lv_session_set_wait_limit(lv_session *s, uint32_t polls)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_set_wait_limit: session is null");
    s->wait_limit = polls;
    return LV_OK;
}

extern "C" int lv_session_timer_start(lv_session *s)
{
    if (!s) return fail(LV_ERR_ARG, "lv_session_timer_start: session is null");
    return timer_start(&s->ev_start, &s->ev_stop, s->stream);
}

extern "C" int lv_session_timer_stop(lv_session *s, float *ms)
{
    if (!s || !ms) return fail(LV_ERR_ARG, "lv_session_timer_stop: null argument");
    LV_TRY(timer_stop(s->ev_start, s->ev_stop, s->stream, ms));
    s->in_flight = false;
    return LV_OK;
}

// -----------------------------------------------------------------------------------------------------------
// cache dump / restore, trace
// -----------------------------------------------------------------------------------------------------------
static int kv_args(const char *who, lv_session *s, uint32_t layer, uint32_t n_tokens, const void *p)
{
    if (!s || (n_tokens && !p)) return fail(LV_ERR_ARG, "%s: null argument", who);
    if (layer >= s->model->hp.layers) return fail(LV_ERR_RANGE, "%s: layer %u of %u", who, layer, s->model->hp.layers);
    if (n_tokens > s->backlog) return fail(LV_ERR_RANGE, "%s: %u rows of a backlog of %u", who, n_tokens, s->backlog);
    if (s->in_flight) return fail(LV_ERR_STATE, "%s: a step is in flight", who);
    return LV_OK;
}

extern "C" int lv_kv_read(lv_session *s, uint32_t layer, int which, uint32_t n_tokens, void *dst)
{
    LV_TRY(kv_args("lv_kv_read", s, layer, n_tokens, dst));
    if (n_tokens == 0) return LV_OK;
    HIP_TRY(hipMemcpyAsync(dst, kv_ptr(s, layer, which), (size_t)n_tokens * s->model->hp.dim * 2, hipMemcpyDeviceToHost, s->stream));
    HIP_TRY(hipStreamSynchronize(s->stream));
    return LV_OK;
}

extern "C" int lv_kv_write(lv_session *s, uint32_t layer, int which, uint32_t n_tokens, const void *src)
{
    LV_TRY(kv_args("lv_kv_write", s, layer, n_tokens, src));
    if (n_tokens == 0) return LV_OK;
    HIP_TRY(hipMemcpyAsync(kv_ptr(s, layer, which), src, (size_t)n_tokens * s->model->hp.dim * 2, hipMemcpyHostToDevice, s->stream));
    HIP_TRY(hipStreamSynchronize(s->stream));
    return LV_OK;
}

extern "C" int lv_trace_enable(lv_session *s, int enable)
{
    if (!s) return fail(LV_ERR_ARG, "lv_trace_enable: session is null");
    if (s->in_flight) return fail(LV_ERR_STATE, "lv_trace_enable: a step is in flight");
    if (enable && !s->trace_buf) {
        HIP_TRY(hipSetDevice(s->model->ctx->device));
        LV_TRY(trace_reserve(s, 1));
        HIP_TRY(hipStreamSynchronize(s->stream));
    }
    s->trace = enable != 0;
    return LV_OK;
}

extern "C" int lv_trace_rows(lv_session *s, uint32_t *rows)
{
    if (!s || !rows) return fail(LV_ERR_ARG, "lv_trace_rows: null argument");
    if (!s->trace || !s->trace_buf) return fail(LV_ERR_STATE, "lv_trace_rows: record mode is off");
    *rows = s->trace_n;
    return LV_OK;
}

extern "C" int lv_trace_read_rows(lv_session *s, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, float *dst)
{
    if (!s || (n_rows && !dst)) return fail(LV_ERR_ARG, "lv_trace_read_rows: null argument");
    if (!s->trace || !s->trace_buf) return fail(LV_ERR_STATE, "lv_trace_read_rows: record mode is off");
    const lv_hparams &hp = s->model->hp;
    if (layer >= hp.layers || which < 0 || which >= LV_TRACE_COUNT) return fail(LV_ERR_RANGE, "lv_trace_read_rows: layer %u / buffer %d", layer, which);
    if (row0 > s->trace_n || n_rows > s->trace_n - row0)
        return fail(LV_ERR_RANGE, "lv_trace_read_rows: rows %u..%u of a step of %u", row0, row0 + n_rows, s->trace_n);
    if (n_rows == 0) return LV_OK;
    HIP_TRY(hipSetDevice(s->model->ctx->device));
    if (which == LV_TRACE_ATTN) {
        if (!s->trace_attn) return fail(LV_ERR_STATE, "lv_trace_read_rows: no attention weights (the cache has no rows)");
        // rows of one layer lie one after the other
        HIP_TRY(hipMemcpyAsync(dst, trace_attn_slot(s, layer, row0), (size_t)n_rows * s->backlog * hp.heads * 4, hipMemcpyDeviceToHost, s->stream));
    } else {
        const size_t slot = hp.dim > hp.ff ? hp.dim : hp.ff, have = which == LV_TRACE_FF ? hp.ff : hp.dim;
        HIP_TRY(hipMemcpy2DAsync(dst, have * 4, trace_slot(s, layer, which, row0), slot * 4, have * 4, n_rows, hipMemcpyDeviceToHost, s->stream));
    }
    return lv_step_wait(s);     // the one place a step ends: stream wait, status word of the persistent kernel, its bookkeeping
}

extern "C" int lv_trace_read(lv_session *s, uint32_t layer, int which, float *dst, uint32_t count)
{
    if (!s || !dst) return fail(LV_ERR_ARG, "lv_trace_read: null argument");
    if (!s->trace || !s->trace_buf) return fail(LV_ERR_STATE, "lv_trace_read: record mode is off");
    const lv_hparams &hp = s->model->hp;
    if (layer >= hp.layers || which < 0 || which >= LV_TRACE_COUNT) return fail(LV_ERR_RANGE, "lv_trace_read: layer %u / buffer %d", layer, which);
    const uint32_t have = which == LV_TRACE_FF ? hp.ff : which == LV_TRACE_ATTN ? s->backlog * hp.heads : hp.dim;
    if (count != have) return fail(LV_ERR_ARG, "lv_trace_read: buffer %d holds %u floats a row, %u asked", which, have, count);
    if (s->trace_n == 0) {
        // nothing recorded yet: the buffers' initial zeros, as before any step
        memset(dst, 0, (size_t)count * 4);
        return LV_OK;
    }
    return lv_trace_read_rows(s, layer, which, s->trace_n - 1, 1, dst);
}
