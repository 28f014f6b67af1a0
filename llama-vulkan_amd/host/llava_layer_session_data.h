// llava_layer_session_data.h — one layer's share of a session: its K and V cache planes and, in record mode,
// its trace buffers.  In the reference this class owns Vulkan buffers (llava_layer_session_data.h:17-45);
// here the memory belongs to the session's HIP arena and this is a typed view of one layer of it.
#pragma once

#include <string>

#include "types.h"

class llava_layer_session_data {
public:
    llava_layer_session_data(llava_session *session, u32 layer);

    // K rows then V rows, token_count rows of `dim` fp16 values each (llava_layer_session_data.cpp:165-172)
    void dump_kv_cache(u8 *dst, u32 token_count);
    void restore_kv_cache(const u8 *src, u32 token_count);
    // appends this layer's record-mode buffers to out_fd in the frame format of llava_buffer.cpp:497-522
    void dump_tracing_layers(int out_fd, const std::string &name);
    // cache resizing is done for all layers at once by the session (lv_session_reserve); kept for interface parity
    void flush_buffers_on_gpu() {}

    llava_session *const session;
    const u32 layer;
};
