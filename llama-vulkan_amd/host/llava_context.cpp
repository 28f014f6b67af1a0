// llava_context.cpp — model load onto the device and the command line front end.
// The reference's run() (llava_context.cpp:151-380) also brings up Vulkan; here device bring-up is lv_ctx_create +
// lv_model_upload.  With -s the loaded model is handed to the token server (server/server.h).
#include "llava_context.h"

#include <csignal>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <vector>

#include "llava_hip.h"
#include "llava_session.h"
#include "server/server.h"

llava_context::llava_context() = default;

llava_context::~llava_context()
{
    if (device_model) lv_model_destroy(device_model);
    if (device_ctx) lv_ctx_destroy(device_ctx);
    delete model;
}

bool llava_context::open_model_file(const std::string &path)
{
    if (model) {
        problem = "a model is already loaded";
        return false;
    }
    ggml_file *file = new ggml_file(path.c_str());
    if (!file->is_open()) {
        problem = file->error();
        delete file;
        return false;
    }
    model = file;
    return true;
}

bool llava_context::load_model(const std::string &path, int device)
{
    if (model) {
        problem = "a model is already loaded";
        return false;
    }
    ggml_file *file = new ggml_file(path.c_str());
    if (!file->is_open()) {
        problem = file->error();
        delete file;
        return false;
    }
    if (lv_ctx_create(device, &device_ctx) != LV_OK) {
        problem = lv_last_error();
        std::cerr << problem << std::endl;
        delete file;
        return false;
    }
    // one table entry per tensor record of the file, straight from the descriptors
    std::vector<lv_tensor_desc> table;
    table.reserve(file->get_tables().size());
    for (const ggml_data_descriptor &d : file->get_tables())
        table.push_back({d.name.c_str(), static_cast<uint32_t>(d.ftype), d.offset, d.shape1, d.shape2, d.size});
    const ggml_header &h = file->get_header();
    const lv_hparams hp = {h.file_version, h.vocab_size, h.dim, h.n_heads, h.n_layers, h.rot, file->get_ff_size()};
    if (lv_model_upload(device_ctx, file->data(), file->data_size(), &hp, table.data(), static_cast<uint32_t>(table.size()), &device_model) != LV_OK) {
        problem = lv_last_error();
        std::cerr << problem << std::endl;
        lv_ctx_destroy(device_ctx);
        device_ctx = nullptr;
        delete file;
        return false;
    }
    model = file;
    return true;
}

// SIGINT / SIGTERM during the token loop end the generation after the current token (llava_context.cpp:352 polls its
// signalfd at the same place)
static volatile std::sig_atomic_t g_interrupted = 0;
static void note_interrupt(int) { g_interrupted = 1; }

static void print_usage(const char *argv0)
{
    std::cerr << "usage: " << argv0 << " [-m|--model FILE] [--print_header] [--greedy] [--seed N] [-n TOKENS] [-d DEVICE] [-v|--verbose] [-h] [PROMPT]\n"
              << "       " << argv0 << " [-m|--model FILE] -s|--server [--port N] [--bind ADDRESS]\n"
              << "       the model path may also come from the LLAVA_MODEL environment variable\n";
}

// Flags of the reference kept: -m/--model, --print_header, -h, -v/--verbose, -c/--control (refused, as there), trailing positional prompt, LLAVA_MODEL
// (llava_context.cpp:163-212).  --use-prebuilt, --debug and --sigdebug concern Vulkan shader builds, the
// validation layer and signalfd debugging and are accepted and ignored.  -s/--server starts the token server after
// the model is loaded (llava_context.cpp:333-336); --port and --bind are additions (the reference listens on 0.0.0.0:1337).
int llava_context::run(int argc, char **argv)
{
    std::string path, prompt;
    bool print_header = false, greedy = false, have_seed = false, server_mode = false;
    u32 seed = 0, max_new = ~0u, port = 1337;
    std::string bind_address = "0.0.0.0";
    int device = 0;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        auto value = [&](const char *flag) -> const char * {
            if (i + 1 >= argc) {
                std::cerr << flag << " needs a value" << std::endl;
                return nullptr;
            }
            return argv[++i];
        };
        if (a == "-h" || a == "--help") { print_usage(argv[0]); return 0; }
        else if (a == "-v" || a == "--verbose") ++verbosity;
        else if (a == "-c" || a == "--control") { std::cerr << "Control disabled for now" << std::endl; return 1; }   // llava_context.cpp:186-187,202-205
        else if (a == "--print_header") print_header = true;
        else if (a == "--greedy") greedy = true;
        else if (a == "--use-prebuilt" || a == "--debug" || a == "--sigdebug") continue;
        else if (a == "-s" || a == "--server") server_mode = true;
        else if (a == "--port") { const char *v = value("--port"); if (!v) return 1; port = static_cast<u32>(std::strtoul(v, nullptr, 0)); }
        else if (a == "--bind") { const char *v = value("--bind"); if (!v) return 1; bind_address = v; }
        else if (a == "-m" || a == "--model") { const char *v = value("--model"); if (!v) return 1; path = v; }
        else if (a == "--seed") { const char *v = value("--seed"); if (!v) return 1; seed = static_cast<u32>(std::strtoul(v, nullptr, 0)); have_seed = true; }
        else if (a == "-n") { const char *v = value("-n"); if (!v) return 1; max_new = static_cast<u32>(std::strtoul(v, nullptr, 0)); }
        else if (a == "-d") { const char *v = value("-d"); if (!v) return 1; device = std::atoi(v); }
        else if (!a.empty() && a[0] == '-') { std::cerr << "Unknown argument " << a << std::endl; print_usage(argv[0]); return 1; }
        else prompt = a;
    }
    if (path.empty()) {
        const char *env = std::getenv("LLAVA_MODEL");
        if (!env) {
            std::cerr << "No model given: use -m FILE or set LLAVA_MODEL" << std::endl;
            return 1;
        }
        path = env;
    }
    // before the device runtime starts its threads: they inherit the mask (llava_context.cpp:284-287 sets up its
    // signalfd at the same point)
    if (server_mode) lsrv::llava_server::block_termination_signals();
    if (!load_model(path, device)) return 1;
    if (print_header) model->print_info();
    if (verbosity) {
        char name[256];
        uint32_t cus = 0;
        uint64_t hbm = 0;
        if (lv_ctx_info(device_ctx, name, sizeof name, &cus, &hbm) == LV_OK)
            std::cout << "Selected device: " << name << ", " << cus << " compute units, " << (hbm >> 30) << " GiB" << std::endl;
    }
    if (server_mode) {
        if (port > 65535) {
            std::cerr << "--port " << port << " is not a TCP port" << std::endl;
            return 1;
        }
        lsrv::llava_server server(this, static_cast<u16>(port), bind_address);
        return server.serve_forever() ? 0 : 1;
    }
    if (prompt.empty()) return 0;

    // the token loop of llava_context.cpp:336-373
    const u32 eos_id = 2;
    llava_session session(this);
    if (have_seed) session.set_sampler_seed(seed);
    if (!session.good() || !session.set_text(prompt)) {
        std::cerr << "[!] System prompt overflows backlog buffer !" << std::endl;
        return 1;
    }
    g_interrupted = 0;
    auto old_int = std::signal(SIGINT, note_interrupt);
    auto old_term = std::signal(SIGTERM, note_interrupt);
    std::cout << prompt << std::flush;
    u32 next = session.predict_next_token(greedy);
    u32 produced = 0;
    while (true) {
        if (~next == 0) {
            std::cerr << "Unknown error" << std::endl;
            break;
        }
        if (g_interrupted || next == eos_id || produced >= max_new) break;
        if (!session.push_token(next)) break;  // context full
        if (!session.start_next_token_prediction()) {
            std::cerr << "Cannot start processing, unknown error" << std::endl;
            break;
        }
        std::cout << model->get_tokens()[next].text << std::flush;  // printed while the device works
        ++produced;
        next = session.finish_next_token_prediction(greedy);
    }
    if (~next != 0 && next != eos_id && produced < max_new) std::cout << model->get_tokens()[next].text;
    std::cout << std::endl;
    std::signal(SIGINT, old_int);
    std::signal(SIGTERM, old_term);
    return 0;
}
