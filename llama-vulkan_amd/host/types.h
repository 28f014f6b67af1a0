// types.h — scalar aliases, GGML element types and return codes of the host surface.
// Values follow the reference (types.h:23-55) because they travel in model files and on the server wire.
#pragma once

#include <cstdint>
#include <string>

using u8 = std::uint8_t;
using u16 = std::uint16_t;
using u32 = std::uint32_t;
using u64 = std::uint64_t;

// element type ids as stored in GGJT tensor records
enum class ggml_value_type : u16 {
    f32 = 0, f16 = 1, q4_0 = 2, q4_1 = 3, q5_0 = 6, q5_1 = 7, q8_0 = 8, q8_1 = 9,
    q2_K = 10, q3_K = 11, q4_K = 12, q5_K = 13, q6_K = 14, q8_K = 15,
};

// result of session-level file operations and of server commands
enum class ReturnCode : u32 {
    ok = 0, nok = 1, no_such_session = 2, tick_already_requested = 3, already_running = 4,
    not_tracing = 5, batched_tick = 6, bad_arguments = 7, unknown_command = 8,
};

class ggml_file;
class llava_context;
class llava_session;
class llava_layer_session_data;
