// llava_session.h — one conversation: token buffer, context ("backlog") sizing, step start/finish, sampling,
// rewind, record mode, snapshot/restore.  Public interface of the reference's class (llava_session.h:39-62)
// with two additions: finish_next_token_prediction() can sample greedily, and the sampler's seed can be fixed.
#pragma once

#include <memory>
#include <random>
#include <string>
#include <vector>

#include "ggml_file.h"
#include "llava_layer_session_data.h"
#include "types.h"

struct lv_session;

// launch geometry the reference derives per session (llava_session.h:15-37); reported for tools that read it
struct specialization_variables_t {
    u32 head_count, quarterrot, backlog, max_wgs, max_wgs_bits, ff_size, softmax_head_per_wavefront, backlog_bits, rot_bits, rot;
    u32 matmul_dim_row_per_wavefront, matmul_dim_row_worker_count, matmul_dim_row_worker_count_log2, matmul_dim_q4_block_count_per_worker,
        matmul_dim_q4_blocks_per_row;
    u32 matmul_ff_row_per_wavefront, matmul_ff_row_worker_count, matmul_ff_row_worker_count_log2, matmul_ff_q4_block_count_per_worker,
        matmul_ff_q4_blocks_per_row;
    u32 batch_enabled;
};

class llava_session {
    friend class llava_layer_session_data;

public:
    explicit llava_session(llava_context *ctx);
    ~llava_session();
    llava_session(const llava_session &) = delete;
    llava_session &operator=(const llava_session &) = delete;

    [[nodiscard]] const std::vector<llava_layer_session_data *> &get_layer_data() const;
    [[nodiscard]] bool set_text(const std::string &new_text);
    [[nodiscard]] bool add_text(const std::string &s);
    [[nodiscard]] bool push_token(u32 token);
    [[nodiscard]] u32 get_token_count() const { return static_cast<u32>(token_buffer.size()); }
    [[nodiscard]] const std::vector<u32> &get_token_buffer() const { return token_buffer; }

    // start = asynchronous submit of every token not yet in the cache; finish = the only wait, then sampling.
    // finish returns ~0U when the device reported an error.  deterministic = greedy (first strict maximum).
    [[nodiscard]] bool start_next_token_prediction();
    [[nodiscard]] u32 finish_next_token_prediction(bool deterministic = false);
    [[nodiscard]] u32 predict_next_token(bool deterministic = false);

    [[nodiscard]] const specialization_variables_t &get_spevar_struct() const { return specialization_variables; }
    [[nodiscard]] bool is_tracing_enabled() const { return options != 0; }

    void rewind(u32 n);
    ReturnCode set_options(u32 new_options);
    ReturnCode save_frame(const std::string &path);
    ReturnCode snapshot(const std::string &path);
    ReturnCode restore(const std::string &path);

    // additions
    // What one stochastic pick went through, for checks of its arithmetic: the tokens that passed the cut with their
    // probabilities (after penalty and temperature, over the whole vocabulary), and which of them was drawn.
    struct sampler_probe {
        std::vector<u32> kept_ids;
        std::vector<float> kept_p;
        float kept_sum = 0.f;
        int pick = -1;
    };
    // The stochastic branch of get_last_predicted_token (llava_session.cpp:154-194) as a function of its inputs: the logits
    // (taken by value, they are overwritten), the token history, the running mu and the generator.
    static u32 sample_token(std::vector<float> p, const u32 *history, std::size_t history_size, float &mu, std::mt19937 &rng, sampler_probe *probe = nullptr);
    void set_sampler_seed(u32 seed);                       // the reference seeds with time(nullptr)
    [[nodiscard]] u32 get_backlog_size() const { return backlog_size; }
    [[nodiscard]] u32 get_tokens_in_gpu() const { return current_tokens_in_gpu; }
    [[nodiscard]] const std::vector<float> &get_last_logits() const { return last_logits; }
    [[nodiscard]] lv_session *get_device_session() const { return device_session; }
    [[nodiscard]] bool good() const { return device_session != nullptr; }

    llava_context *const ctx;
    const ggml_file *const model;

private:
    [[nodiscard]] u32 get_last_predicted_token(bool deterministic);
    [[nodiscard]] bool set_backlog_size(u32 new_size);
    void recreate_spevars();
    void step_failed();
    bool settle_step();

    // sampler state and constants (llava_session.h:68-77)
    std::mt19937 rng;
    static constexpr u32 repeat_last_n = 64;
    static constexpr float repeat_penalty = 1.1f, alpha_frequency = 0.1f, alpha_presence = 0.0f, temp = 0.8f, mirostat_tau = 5.0f, mirostat_eta = 0.1f;
    float mirostat_mu;

    lv_session *device_session = nullptr;
    std::vector<llava_layer_session_data *> layer_data;
    std::vector<u32> token_buffer;
    std::vector<float> last_logits;
    u32 current_tokens_in_gpu = 0;
    u32 backlog_size;
    u32 batch_size = 0;
    u32 options = 0;
    bool step_in_flight = false;
    u32 step_first_row = 0;  // first cache row of the step that was started last
    specialization_variables_t specialization_variables{};
};
