// capi.cpp — flat C view of the host classes for callers that cannot include C++ headers (the Python tests).
// Not a second interface: every function forwards to one public method of ggml_file / llava_context /
// llava_session and adds nothing.
#include <cstring>
#include <exception>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "ggml_file.h"
#include "llava_context.h"
#include "llava_session.h"
#include "server/server.h"

namespace {
unsigned copy_out(const std::string &s, char *out, unsigned cap)
{
    const unsigned n = static_cast<unsigned>(s.size());
    if (out && cap) std::memcpy(out, s.data(), n < cap ? n : cap);
    return n;
}
}  // namespace

extern "C" {

// ---- ggml_file ------------------------------------------------------------------------------------------
// null only when the object itself cannot be allocated; a bad file gives an object that is not open
void *llh_file_open(const char *path)
{
    try {
        return new ggml_file(path);
    } catch (const std::exception &) {
        return nullptr;
    }
}
void llh_file_close(void *f) { delete static_cast<ggml_file *>(f); }
int llh_file_is_open(void *f) { return static_cast<ggml_file *>(f)->is_open(); }
unsigned llh_file_error(void *f, char *out, unsigned cap) { return copy_out(static_cast<ggml_file *>(f)->error(), out, cap); }
// out[0..9]: file_version, vocab_size, dim, multiple_of, n_heads, n_layers, rot, ftype, ff_size, tensor count
void llh_file_header(void *f, unsigned *out)
{
    const ggml_file *g = static_cast<ggml_file *>(f);
    const ggml_header &h = g->get_header();
    const unsigned v[10] = {h.file_version, h.vocab_size, h.dim, h.multiple_of, h.n_heads, h.n_layers, h.rot, h.ftype, g->get_ff_size(),
                            static_cast<unsigned>(g->get_tables().size())};
    std::memcpy(out, v, sizeof v);
}
void llh_file_print_info(void *f) { static_cast<ggml_file *>(f)->print_info(); }
// tensor by table index; returns the name length
unsigned llh_file_tensor_at(void *f, unsigned index, char *name, unsigned cap, unsigned *ftype, unsigned long long *offset, unsigned *shape1,
                            unsigned *shape2, unsigned long long *size)
{
    const ggml_data_descriptor &d = static_cast<ggml_file *>(f)->get_tables().at(index);
    *ftype = static_cast<unsigned>(d.ftype); *offset = d.offset; *shape1 = d.shape1; *shape2 = d.shape2; *size = d.size;
    return copy_out(d.name, name, cap);
}
// tensor by name with the ".weight" fallback; 0 when found
int llh_file_tensor(void *f, const char *name, unsigned *ftype, unsigned long long *offset, unsigned *shape1, unsigned *shape2,
                    unsigned long long *size)
{
    const ggml_data_descriptor *d = static_cast<ggml_file *>(f)->find_buffer_descriptor(name);
    if (!d) return -1;
    *ftype = static_cast<unsigned>(d->ftype); *offset = d->offset; *shape1 = d->shape1; *shape2 = d->shape2; *size = d->size;
    return 0;
}
unsigned llh_file_token(void *f, unsigned id, char *out, unsigned cap, float *score)
{
    const ggml_token &t = static_cast<ggml_file *>(f)->get_tokens().at(id);
    if (score) *score = t.score;
    return copy_out(t.text, out, cap);
}
unsigned llh_file_tokenize(void *f, const char *text, unsigned len, int bos, unsigned *out, unsigned cap)
{
    std::vector<u32> ids;
    static_cast<ggml_file *>(f)->tokenize(ids, std::string(text, len), bos != 0);
    for (size_t i = 0; i < ids.size() && i < cap; ++i) out[i] = ids[i];
    return static_cast<unsigned>(ids.size());
}
unsigned llh_file_detokenize(void *f, const unsigned *ids, unsigned n, char *out, unsigned cap)
{
    return copy_out(static_cast<ggml_file *>(f)->tokens_to_text(ids, n), out, cap);
}

// ---- llava_context ----------------------------------------------------------------------------------------
void *llh_context_new() { return new llava_context; }
void llh_context_free(void *c) { delete static_cast<llava_context *>(c); }
// no C++ exception leaves this file: a load that throws (allocation failure) is a failed load
int llh_context_load(void *c, const char *path, int device)
{
    try {
        return static_cast<llava_context *>(c)->load_model(path, device) ? 0 : -1;
    } catch (const std::exception &) {
        return -1;
    }
}
unsigned llh_context_error(void *c, char *out, unsigned cap) { return copy_out(static_cast<llava_context *>(c)->last_error(), out, cap); }
int llh_context_run(void *c, int argc, char **argv) { return static_cast<llava_context *>(c)->run(argc, argv); }
int llh_context_open_file(void *c, const char *path)
{
    try {
        return static_cast<llava_context *>(c)->open_model_file(path) ? 0 : -1;
    } catch (const std::exception &) {
        return -1;
    }
}

// ---- lsrv::llava_server: open() + serve_forever() on a thread of its own ----------------------------------
struct llh_server {
    lsrv::llava_server server;
    std::thread loop;
    llh_server(llava_context *c, unsigned short port, const char *bind) : server(c, port, bind) {}
};
// null when the socket cannot be opened
void *llh_server_start(void *c, unsigned short port, const char *bind_address)
{
    llh_server *s = new llh_server(static_cast<llava_context *>(c), port, bind_address);
    if (!s->server.open()) {
        delete s;
        return nullptr;
    }
    s->loop = std::thread([s] { s->server.serve_forever(); });
    return s;
}
unsigned llh_server_port(void *s) { return static_cast<llh_server *>(s)->server.bound_port(); }
void llh_server_stop(void *h)
{
    llh_server *s = static_cast<llh_server *>(h);
    s->server.request_stop();
    s->loop.join();
    delete s;
}

// ---- llava_session ----------------------------------------------------------------------------------------
void *llh_session_new(void *c) { return new llava_session(static_cast<llava_context *>(c)); }
void llh_session_free(void *s) { delete static_cast<llava_session *>(s); }
int llh_session_good(void *s) { return static_cast<llava_session *>(s)->good(); }
int llh_session_set_text(void *s, const char *t, unsigned n) { return static_cast<llava_session *>(s)->set_text(std::string(t, n)); }
int llh_session_add_text(void *s, const char *t, unsigned n) { return static_cast<llava_session *>(s)->add_text(std::string(t, n)); }
int llh_session_push_token(void *s, unsigned t) { return static_cast<llava_session *>(s)->push_token(t); }
unsigned llh_session_token_count(void *s) { return static_cast<llava_session *>(s)->get_token_count(); }
unsigned llh_session_tokens(void *s, unsigned *out, unsigned cap)
{
    const std::vector<u32> &b = static_cast<llava_session *>(s)->get_token_buffer();
    for (size_t i = 0; i < b.size() && i < cap; ++i) out[i] = b[i];
    return static_cast<unsigned>(b.size());
}
int llh_session_start(void *s) { return static_cast<llava_session *>(s)->start_next_token_prediction(); }
unsigned llh_session_finish(void *s, int deterministic) { return static_cast<llava_session *>(s)->finish_next_token_prediction(deterministic != 0); }
unsigned llh_session_predict(void *s, int deterministic) { return static_cast<llava_session *>(s)->predict_next_token(deterministic != 0); }
void llh_session_rewind(void *s, unsigned n) { static_cast<llava_session *>(s)->rewind(n); }
unsigned llh_session_set_options(void *s, unsigned o) { return static_cast<unsigned>(static_cast<llava_session *>(s)->set_options(o)); }
int llh_session_is_tracing(void *s) { return static_cast<llava_session *>(s)->is_tracing_enabled(); }
unsigned llh_session_save_frame(void *s, const char *p) { return static_cast<unsigned>(static_cast<llava_session *>(s)->save_frame(p)); }
unsigned llh_session_snapshot(void *s, const char *p) { return static_cast<unsigned>(static_cast<llava_session *>(s)->snapshot(p)); }
unsigned llh_session_restore(void *s, const char *p) { return static_cast<unsigned>(static_cast<llava_session *>(s)->restore(p)); }
void llh_session_seed(void *s, unsigned seed) { static_cast<llava_session *>(s)->set_sampler_seed(seed); }
// llava_session::sample_token on caller-supplied logits: returns the token; *mu is read and updated; kept_ids / kept_p
// receive up to cap entries of the kept set, *kept_count its size, *kept_sum its probability mass, *pick the drawn index
unsigned llh_sample_token(const float *logits, unsigned n_vocab, const unsigned *history, unsigned history_size, float *mu, unsigned seed,
                          unsigned *kept_ids, float *kept_p, unsigned cap, unsigned *kept_count, float *kept_sum, int *pick)
{
    std::mt19937 rng(seed);
    llava_session::sampler_probe probe;
    const unsigned token = llava_session::sample_token(std::vector<float>(logits, logits + n_vocab), history, history_size, *mu, rng, &probe);
    const unsigned n = static_cast<unsigned>(probe.kept_ids.size());
    for (unsigned i = 0; i < n && i < cap; ++i) {
        kept_ids[i] = probe.kept_ids[i];
        kept_p[i] = probe.kept_p[i];
    }
    *kept_count = n;
    *kept_sum = probe.kept_sum;
    *pick = probe.pick;
    return token;
}
// the lv_session the object drives, for calls of the device library that the class does not wrap
void *llh_session_device(void *s) { return static_cast<llava_session *>(s)->get_device_session(); }
unsigned llh_session_backlog(void *s) { return static_cast<llava_session *>(s)->get_backlog_size(); }
unsigned llh_session_tokens_in_gpu(void *s) { return static_cast<llava_session *>(s)->get_tokens_in_gpu(); }
unsigned llh_session_logits(void *s, float *out, unsigned cap)
{
    const std::vector<float> &l = static_cast<llava_session *>(s)->get_last_logits();
    if (out) std::memcpy(out, l.data(), sizeof(float) * (l.size() < cap ? l.size() : cap));
    return static_cast<unsigned>(l.size());
}
// out[0..20]: the launch geometry struct of get_spevar_struct()
void llh_session_spevars(void *s, unsigned *out) { std::memcpy(out, &static_cast<llava_session *>(s)->get_spevar_struct(), sizeof(specialization_variables_t)); }
unsigned llh_session_layer_count(void *s) { return static_cast<unsigned>(static_cast<llava_session *>(s)->get_layer_data().size()); }
}
