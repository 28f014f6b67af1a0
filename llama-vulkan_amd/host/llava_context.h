// llava_context.h — process-wide state the sessions share: the parsed model file, the HIP device context and
// the uploaded weights.  Stands where the reference keeps its Vulkan instance/device/queue/pools and layer
// objects (llava_context.h:15-86); what is left of that class is get_model() and run().
#pragma once

#include <mutex>
#include <string>

#include "ggml_file.h"
#include "types.h"

struct lv_ctx;
struct lv_model;

class llava_context {
public:
    llava_context();
    ~llava_context();
    llava_context(const llava_context &) = delete;
    llava_context &operator=(const llava_context &) = delete;

    // Command line front end (llava_context.cpp:151-380): flags, model load, prompt evaluation, token loop.
    int run(int argc, char **argv);

    // Opens and uploads a model without going through argv.  False + message on stderr when anything fails.
    bool load_model(const std::string &path, int device = 0);
    // Opens and parses the file only: vocabulary and tensor table are available, sessions are not (for tools that
    // run without a device).
    bool open_model_file(const std::string &path);

    [[nodiscard]] const ggml_file *get_model() const { return model; }
    [[nodiscard]] lv_ctx *get_device_context() const { return device_ctx; }
    [[nodiscard]] lv_model *get_device_model() const { return device_model; }
    [[nodiscard]] const std::string &last_error() const { return problem; }

    // the reference's device limit used to derive launch geometry (llava_context.cpp:259); kept for
    // get_spevar_struct(), which reports the geometry the reference would have used
    u32 workgroup_size = 1024;
    int verbosity = 0;

private:
    ggml_file *model = nullptr;
    lv_ctx *device_ctx = nullptr;
    lv_model *device_model = nullptr;
    std::string problem;
};
