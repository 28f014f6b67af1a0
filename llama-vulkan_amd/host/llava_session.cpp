// llava_session.cpp — session logic over the lv_* C-ABI.  Behaviour follows the reference's llava_session.cpp
// (cited per function); the device objects it manipulates there are one lv_session handle here.
#include "llava_session.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <ctime>
#include <fcntl.h>
#include <iostream>
#include <map>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "llava_context.h"
#include "llava_hip.h"
#include "utils.h"

namespace {

// llava_session.cpp:23-24: the context grows by doubling between these bounds
constexpr u32 kMinBacklog = 128;
constexpr u32 kMaxBacklog = 2048;

// record-mode buffers in the order they are dumped, with the names the reference gives them
// (llava_layer_session_data.cpp:80-85)
enum class TraceShape { dim, ff, attn };
struct TraceSlot { int which; const char *name; TraceShape shape; };
constexpr TraceSlot kTraceSlots[] = {
    {LV_TRACE_ATTN, "attn_result", TraceShape::attn},
    {LV_TRACE_FF, "ff_result", TraceShape::ff},
    {LV_TRACE_NORM_IN, "normalized_input_logit", TraceShape::dim},
    {LV_TRACE_POST_ATTN, "post_attn_logit", TraceShape::dim},
    {LV_TRACE_POST_ATTN_NORM, "post_attn_norm_logit", TraceShape::dim},
    {LV_TRACE_OUT, "output_logit", TraceShape::dim},
};

// RAII for a file descriptor
struct Fd {
    int fd;
    explicit Fd(int f) : fd(f) {}
    ~Fd() { if (fd >= 0 && ::close(fd) < 0) std::perror("close"); }
    Fd(const Fd &) = delete;
    Fd &operator=(const Fd &) = delete;
};

}  // namespace

// ---------------------------------------------------------------------------------------------------------------
// layer view
// ---------------------------------------------------------------------------------------------------------------
llava_layer_session_data::llava_layer_session_data(llava_session *s, u32 l) : session(s), layer(l) {}

void llava_layer_session_data::dump_kv_cache(u8 *dst, u32 token_count)
{
    const std::size_t plane = static_cast<std::size_t>(token_count) * session->model->get_header().dim * 2;
    if (lv_kv_read(session->device_session, layer, 0, token_count, dst) != LV_OK ||
        lv_kv_read(session->device_session, layer, 1, token_count, dst + plane) != LV_OK)
        std::cerr << "dump_kv_cache: " << lv_last_error() << std::endl;
}

void llava_layer_session_data::restore_kv_cache(const u8 *src, u32 token_count)
{
    const std::size_t plane = static_cast<std::size_t>(token_count) * session->model->get_header().dim * 2;
    if (lv_kv_write(session->device_session, layer, 0, token_count, src) != LV_OK ||
        lv_kv_write(session->device_session, layer, 1, token_count, src + plane) != LV_OK)
        std::cerr << "restore_kv_cache: " << lv_last_error() << std::endl;
}

// One buffer of a frame (llava_buffer.cpp:497-522): u32 shape0, u32 shape1, u32 type, name, zero padding up to a
// multiple of 32 bytes, then the raw fp32 values.
void llava_layer_session_data::dump_tracing_layers(int out_fd, const std::string &name)
{
    const u32 dim = session->model->get_header().dim, ff = session->model->get_ff_size(), heads = session->model->get_header().n_heads;
    // the rows of the last recorded step; before the first one the reference has no trace buffers at all
    // (llava_layer_session_data.cpp:79) and writes nothing
    u32 rows = 0;
    if (lv_trace_rows(session->device_session, &rows) != LV_OK) {
        std::cerr << "dump_tracing_layers: " << lv_last_error() << std::endl;
        return;
    }
    if (rows == 0) return;
    for (const TraceSlot &slot : kTraceSlots) {
        // shape as the reference's buffers have it: (values per row, rows); attn_result is (backlog, heads x rows).  In
        // memory both are one row of the step after the other.
        const u32 shape0 = slot.shape == TraceShape::ff ? ff : slot.shape == TraceShape::attn ? session->backlog_size : dim;
        const u32 shape1 = slot.shape == TraceShape::attn ? heads * rows : rows;
        const std::size_t count = static_cast<std::size_t>(shape0) * shape1;
        std::vector<float> values(count);
        if (lv_trace_read_rows(session->device_session, layer, slot.which, 0, rows, values.data()) != LV_OK) {
            std::cerr << "dump_tracing_layers: " << lv_last_error() << std::endl;
            return;
        }
        const std::string full = name + "." + slot.name;
        const u32 header_size = static_cast<u32>((12 + full.size() + 1 + 31) & ~static_cast<std::size_t>(31));
        std::vector<u8> head(header_size, 0);
        const u32 fields[3] = {shape0, shape1, static_cast<u32>(ggml_value_type::f32)};
        std::memcpy(head.data(), fields, sizeof fields);
        std::memcpy(head.data() + 12, full.data(), full.size());
        if (write_noshort(out_fd, head.data(), head.size()) != head.size() ||
            write_noshort(out_fd, values.data(), values.size() * 4) != values.size() * 4)
            return;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// construction
// ---------------------------------------------------------------------------------------------------------------
llava_session::llava_session(llava_context *_ctx)
    : ctx(_ctx), model(_ctx->get_model()), rng(static_cast<u32>(std::time(nullptr))), mirostat_mu(2 * mirostat_tau), backlog_size(kMinBacklog)
{
    if (!model || !ctx->get_device_model()) {
        std::cerr << "llava_session: the context has no model loaded" << std::endl;
        return;
    }
    if (lv_session_create(ctx->get_device_model(), &device_session) != LV_OK ||
        lv_session_reserve(device_session, backlog_size) != LV_OK) {
        std::cerr << "llava_session: " << lv_last_error() << std::endl;
        if (device_session) lv_session_destroy(device_session);
        device_session = nullptr;
        return;
    }
    for (u32 i = 0; i < model->get_header().n_layers; ++i) layer_data.push_back(new llava_layer_session_data(this, i));
    recreate_spevars();
}

llava_session::~llava_session()
{
    for (llava_layer_session_data *l : layer_data) delete l;
    if (device_session) lv_session_destroy(device_session);
}

const std::vector<llava_layer_session_data *> &llava_session::get_layer_data() const { return layer_data; }

void llava_session::set_sampler_seed(u32 seed)
{
    rng.seed(seed);
    mirostat_mu = 2 * mirostat_tau;
}

// ---------------------------------------------------------------------------------------------------------------
// token buffer and context size
// ---------------------------------------------------------------------------------------------------------------

// llava_session.cpp:303-327
bool llava_session::set_backlog_size(u32 new_size)
{
    if (new_size > kMaxBacklog) return false;
    if (new_size == backlog_size) return true;
    if (new_size < kMinBacklog || new_size < current_tokens_in_gpu) return false;
    settle_step();
    if (lv_session_reserve(device_session, new_size) != LV_OK) {
        std::cerr << "set_backlog_size: " << lv_last_error() << std::endl;
        return false;
    }
    backlog_size = new_size;
    recreate_spevars();
    return true;
}

// llava_session.cpp:257-277.  The reference compares the old token ids with the *characters* of the new text
// when it looks for a reusable prefix (line 271), which almost never matches; here the old tokens are compared
// with the new tokens, so a shared prefix keeps its cache rows.  The resulting logits are the same either way.
bool llava_session::set_text(const std::string &new_text)
{
    if (!good()) return false;
    std::vector<u32> fresh;
    model->tokenize(fresh, new_text, true);
    u32 wanted = backlog_size;
    while (fresh.size() > wanted) wanted <<= 1;
    if (wanted > kMaxBacklog || !set_backlog_size(wanted)) return false;
    u32 keep = 0;
    while (keep < fresh.size() && keep < token_buffer.size() && keep < current_tokens_in_gpu && token_buffer[keep] == fresh[keep]) ++keep;
    // the last token of the new text is always evaluated again: the logits on the device then belong to this text, also
    // when it is a prefix of what was evaluated before (the reference re-evaluates in that case too)
    if (!fresh.empty() && keep == fresh.size()) --keep;
    token_buffer = std::move(fresh);
    current_tokens_in_gpu = keep;
    return true;
}

// llava_session.cpp:279-282
bool llava_session::add_text(const std::string &s)
{
    return set_text(model->tokens_to_text(token_buffer.data(), static_cast<u32>(token_buffer.size())) + s);
}

// llava_session.cpp:284-297
bool llava_session::push_token(u32 token)
{
    if (!good() || token >= model->get_tokens().size()) return false;
    if (token_buffer.size() == backlog_size) {
        if (backlog_size == kMaxBacklog || !set_backlog_size(backlog_size * 2)) return false;
    }
    token_buffer.push_back(token);
    return true;
}

// llava_session.cpp:390-395
void llava_session::rewind(u32 n)
{
    if (n < token_buffer.size()) {
        token_buffer.resize(n);
        current_tokens_in_gpu = std::min(n, current_tokens_in_gpu);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// one step
// ---------------------------------------------------------------------------------------------------------------

// llava_session.cpp:197-229
bool llava_session::start_next_token_prediction()
{
    if (!good()) return false;
    settle_step();  // a caller that starts twice without finishing: the reference would hit its fence too
    const u32 to_process = static_cast<u32>(token_buffer.size()) - current_tokens_in_gpu;
    if (to_process == 0) {
        std::cerr << "GPU is already in sync" << std::endl;
        return false;
    }
    if (token_buffer.size() > backlog_size) {
        std::cerr << "Token buffer overflow" << std::endl;
        return false;
    }
    if (batch_size != to_process) {
        batch_size = to_process;
        recreate_spevars();
    }
    if (lv_step_begin(device_session, token_buffer.data() + current_tokens_in_gpu, to_process, current_tokens_in_gpu) != LV_OK) {
        std::cerr << "start_next_token_prediction: " << lv_last_error() << std::endl;
        return false;
    }
    step_in_flight = true;
    step_first_row = current_tokens_in_gpu;
    current_tokens_in_gpu += to_process;
    return true;
}

// The rows a step writes count as evaluated from the moment it is submitted.  When the step turns out to have failed
// (the device reports an error at the wait), they hold nothing usable: count them as pending again, so that the next
// start evaluates the same tokens into the same rows.
void llava_session::step_failed()
{
    current_tokens_in_gpu = std::min(current_tokens_in_gpu, step_first_row);
}

// waits for a step that was started and never finished; false when that step failed
bool llava_session::settle_step()
{
    if (!step_in_flight) return true;
    step_in_flight = false;
    if (lv_step_wait(device_session) == LV_OK) return true;
    std::cerr << "step failed: " << lv_last_error() << std::endl;
    step_failed();
    return false;
}

// llava_session.cpp:231-234; the reference always samples stochastically here
u32 llava_session::finish_next_token_prediction(bool deterministic)
{
    if (!good()) return ~0u;
    return get_last_predicted_token(deterministic);
}

// llava_session.cpp:236-241
u32 llava_session::predict_next_token(bool deterministic)
{
    if (!start_next_token_prediction()) return ~0u;
    return finish_next_token_prediction(deterministic);
}

// llava_session.cpp:114-195
u32 llava_session::get_last_predicted_token(bool deterministic)
{
    const u32 n_vocab = model->get_header().vocab_size;
    last_logits.resize(n_vocab);
    const int rc = lv_logits_read(device_session, last_logits.data());  // waits for the step
    const bool was_in_flight = step_in_flight;
    step_in_flight = false;
    if (rc != LV_OK) {
        std::cerr << "finish_next_token_prediction: " << lv_last_error() << std::endl;
        if (was_in_flight) step_failed();
        return ~0u;
    }
    std::vector<float> p(last_logits);
    for (float v : p)
        if (std::isnan(v) || std::isinf(v)) {
            std::cerr << "NaN in output buffer" << std::endl;
            break;
        }

    if (deterministic) {  // first strict maximum (:144-152)
        u32 best = 0;
        for (u32 t = 0; t < n_vocab; ++t)
            if (p[t] > p[best]) best = t;
        return best;
    }

    return sample_token(std::move(p), token_buffer.data(), token_buffer.size(), mirostat_mu, rng);
}

// llava_session.cpp:154-194
u32 llava_session::sample_token(std::vector<float> p, const u32 *history, std::size_t history_size, float &mu, std::mt19937 &rng, sampler_probe *probe)
{
    const u32 n_vocab = static_cast<u32>(p.size());
    // repetition / frequency penalty, applied to the newline token only (:157-167)
    std::map<u32, u32> recent;
    const std::size_t from = history_size > repeat_last_n ? history_size - repeat_last_n : 0;
    for (std::size_t i = from; i < history_size; ++i) recent[history[i]]++;
    const auto nl = recent.find(13);
    if (nl != recent.end() && 13 < n_vocab) {
        float &l = p[13];
        l = l <= 0 ? l * repeat_penalty : l / repeat_penalty;
        l -= alpha_frequency * static_cast<float>(nl->second) + alpha_presence;
    }

    // temperature softmax without max subtraction (:169-173)
    float total = 0.f;
    for (u32 t = 0; t < n_vocab; ++t) {
        p[t] = std::exp(p[t] / temp);
        total += p[t];
    }
    // keep what is at least 2^-mu likely (:175-188)
    const float cut = std::pow(0.5f, mu);
    std::vector<u32> ids;
    std::vector<float> kept;
    float kept_sum = 0.f;
    u32 likeliest = 0;
    for (u32 t = 0; t < n_vocab; ++t) {
        p[t] /= total;
        if (p[t] > p[likeliest]) likeliest = t;
        if (p[t] >= cut) {
            kept_sum += p[t];
            kept.push_back(p[t]);
            ids.push_back(t);
        }
    }
    if (probe) {
        probe->kept_ids = ids;
        probe->kept_p = kept;
        probe->kept_sum = kept_sum;
        probe->pick = -1;
    }
    if (ids.empty()) return likeliest;  // nothing passes the cut: the reference would index an empty vector here
    std::discrete_distribution<> dist(kept.begin(), kept.end());
    const int pick = dist(rng);
    if (probe) probe->pick = pick;
    mu += mirostat_eta * (mirostat_tau + std::log2(kept[pick] / kept_sum));  // (:193)
    return ids[pick];
}

// llava_session.cpp:339-388: the launch geometry the reference would use; informational here
void llava_session::recreate_spevars()
{
    specialization_variables_t &sv = specialization_variables;
    const ggml_header &h = model->get_header();
    const u32 wgs = ctx->workgroup_size, ff = model->get_ff_size();
    sv = {};
    sv.head_count = h.n_heads;
    sv.rot = h.rot;
    sv.quarterrot = h.rot / 4;
    sv.rot_bits = ulog2(h.rot);
    sv.max_wgs = wgs;
    sv.max_wgs_bits = ulog2(wgs);
    sv.ff_size = ff;
    sv.matmul_dim_row_worker_count = h.dim == 5120 ? 32 : 128;
    sv.matmul_dim_row_per_wavefront = wgs / sv.matmul_dim_row_worker_count;
    sv.matmul_dim_row_worker_count_log2 = ulog2(sv.matmul_dim_row_worker_count);
    sv.matmul_dim_q4_blocks_per_row = h.dim / 32;
    sv.matmul_dim_q4_block_count_per_worker = static_cast<u32>(updiv(sv.matmul_dim_q4_blocks_per_row, sv.matmul_dim_row_worker_count));
    sv.matmul_ff_row_worker_count = 128;
    sv.matmul_ff_row_per_wavefront = wgs / sv.matmul_ff_row_worker_count;
    sv.matmul_ff_row_worker_count_log2 = ulog2(sv.matmul_ff_row_worker_count);
    sv.matmul_ff_q4_blocks_per_row = ff / 32;
    sv.matmul_ff_q4_block_count_per_worker = static_cast<u32>(updiv(sv.matmul_ff_q4_blocks_per_row, sv.matmul_dim_row_worker_count));
    sv.backlog = backlog_size;
    sv.softmax_head_per_wavefront = wgs / backlog_size;
    sv.backlog_bits = ulog2(backlog_size);
    sv.batch_enabled = batch_size > 1 ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------------------------
// record mode
// ---------------------------------------------------------------------------------------------------------------

// llava_session.cpp:403-418: any non-zero value switches recording on
ReturnCode llava_session::set_options(u32 new_options)
{
    if (options == new_options) return ReturnCode::ok;
    if (!good()) return ReturnCode::nok;
    settle_step();
    if (lv_trace_enable(device_session, new_options != 0) != LV_OK) return ReturnCode::nok;
    options = new_options;
    return ReturnCode::ok;
}

// llava_session.cpp:424-445
ReturnCode llava_session::save_frame(const std::string &path)
{
    if (!is_tracing_enabled()) return ReturnCode::not_tracing;
    Fd out(::open(path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644));
    if (out.fd < 0) {
        std::perror("open");
        return ReturnCode::nok;
    }
    u32 i = 0;
    for (llava_layer_session_data *l : layer_data) l->dump_tracing_layers(out.fd, "layer." + std::to_string(i++));
    return ReturnCode::ok;
}

// ---------------------------------------------------------------------------------------------------------------
// snapshot / restore: u32 n, u32 tokens[n], then per layer K f16[n][dim] followed by V f16[n][dim]
// (llava_session.cpp:447-603, llava_layer_session_data.cpp:165-181)
// ---------------------------------------------------------------------------------------------------------------
ReturnCode llava_session::snapshot(const std::string &path)
{
    if (!good()) return ReturnCode::nok;
    settle_step();
    const u32 n = current_tokens_in_gpu, dim = model->get_header().dim;
    const std::size_t per_layer = static_cast<std::size_t>(2) * n * dim * 2;
    const std::size_t total = layer_data.size() * per_layer + 4 * static_cast<std::size_t>(n) + 4;
    Fd out(::open(path.c_str(), O_RDWR | O_CREAT | O_TRUNC, 0644));
    if (out.fd < 0) {
        std::perror("open");
        return ReturnCode::nok;
    }
    if (ftruncate(out.fd, static_cast<off_t>(total)) < 0) {
        std::perror("ftruncate");
        return ReturnCode::nok;
    }
    void *map = mmap(nullptr, total, PROT_READ | PROT_WRITE, MAP_SHARED, out.fd, 0);
    if (map == MAP_FAILED) {
        std::perror("mmap");
        return ReturnCode::nok;
    }
    u8 *bytes = static_cast<u8 *>(map);
    std::memcpy(bytes, &n, 4);
    if (n) std::memcpy(bytes + 4, token_buffer.data(), static_cast<std::size_t>(n) * 4);
    u8 *cursor = bytes + 4 + static_cast<std::size_t>(n) * 4;
    for (llava_layer_session_data *l : layer_data) {
        l->dump_kv_cache(cursor, n);
        cursor += per_layer;
    }
    if (msync(map, total, MS_SYNC) < 0) std::perror("msync");
    if (munmap(map, total) < 0) std::perror("munmap");
    return ReturnCode::ok;
}

ReturnCode llava_session::restore(const std::string &path)
{
    if (!good()) return ReturnCode::nok;
    Fd in(::open(path.c_str(), O_RDONLY));
    if (in.fd < 0) {
        std::perror("open");
        return ReturnCode::nok;
    }
    struct stat st{};
    if (fstat(in.fd, &st) < 0) {
        std::perror("fstat");
        return ReturnCode::nok;
    }
    if (!S_ISREG(st.st_mode)) {
        std::cerr << "Expected regular file got something else" << std::endl;
        return ReturnCode::nok;
    }
    if (st.st_size < 4) {
        std::cerr << "File too short" << std::endl;
        return ReturnCode::nok;
    }
    const std::size_t size = static_cast<std::size_t>(st.st_size);
    void *map = mmap(nullptr, size, PROT_READ, MAP_SHARED, in.fd, 0);
    if (map == MAP_FAILED) {
        std::perror("mmap");
        return ReturnCode::nok;
    }
    struct Unmap { void *p; std::size_t n; ~Unmap() { if (munmap(p, n) < 0) std::perror("munmap"); } } unmap{map, size};
    const u8 *bytes = static_cast<const u8 *>(map);
    u32 n;
    std::memcpy(&n, bytes, 4);
    if (n > kMaxBacklog) {
        std::cerr << "Too many tokens" << std::endl;
        return ReturnCode::nok;
    }
    const u32 dim = model->get_header().dim;
    const std::size_t per_layer = static_cast<std::size_t>(2) * n * dim * 2;
    if (layer_data.size() * per_layer + 4 * static_cast<std::size_t>(n) + 4 != size) {
        std::cerr << "File size mismatch" << std::endl;
        return ReturnCode::nok;
    }
    std::vector<u32> toks(n);
    if (n) std::memcpy(toks.data(), bytes + 4, static_cast<std::size_t>(n) * 4);
    for (u32 t : toks)
        if (t >= model->get_tokens().size()) {
            std::cerr << "Token id outside the vocabulary" << std::endl;
            return ReturnCode::nok;
        }
    u32 needed = kMinBacklog;
    while (needed < n) needed <<= 1;
    settle_step();
    rewind(0);
    if (!set_backlog_size(needed)) {
        std::cerr << "Cannot set backlog size" << std::endl;
        return ReturnCode::nok;
    }
    token_buffer = std::move(toks);
    current_tokens_in_gpu = n;
    const u8 *cursor = bytes + 4 + static_cast<std::size_t>(n) * 4;
    for (llava_layer_session_data *l : layer_data) {
        l->restore_kv_cache(cursor, n);
        cursor += per_layer;
    }
    return ReturnCode::ok;
}
