#include "utils.h"

#include <cerrno>
#include <cstdio>
#include <unistd.h>

const char *ftype_name(ggml_value_type type)
{
    struct Entry { ggml_value_type id; const char *text; };
    static const Entry table[] = {
        {ggml_value_type::f32, "f32"},   {ggml_value_type::f16, "f16"},   {ggml_value_type::q4_0, "q4_0"}, {ggml_value_type::q4_1, "q4_1"},
        {ggml_value_type::q5_0, "q5_0"}, {ggml_value_type::q5_1, "q5_1"}, {ggml_value_type::q8_0, "q8_0"}, {ggml_value_type::q8_1, "q8_1"},
        {ggml_value_type::q2_K, "q2_K"}, {ggml_value_type::q3_K, "q3_K"}, {ggml_value_type::q4_K, "q4_K"}, {ggml_value_type::q5_K, "q5_K"},
        {ggml_value_type::q6_K, "q6_K"}, {ggml_value_type::q8_K, "q8_K"},
    };
    for (const Entry &e : table)
        if (e.id == type) return e.text;
    return nullptr;
}

u32 ulog2(u32 n)
{
    if (n == 0 || (n & (n - 1)) != 0) return ~0u;
    u32 bits = 0;
    while (n > 1) { n >>= 1; ++bits; }
    return bits;
}

bool starts_with(const std::string &text, const std::string &prefix)
{
    return text.size() >= prefix.size() && text.compare(0, prefix.size(), prefix) == 0;
}

bool ends_with(const std::string &text, const std::string &suffix)
{
    return text.size() >= suffix.size() && text.compare(text.size() - suffix.size(), suffix.size(), suffix) == 0;
}

std::size_t read_noshort(int fd, void *dst, std::size_t size)
{
    std::size_t done = 0;
    while (done < size) {
        const ssize_t got = ::read(fd, static_cast<u8 *>(dst) + done, size - done);
        if (got < 0 && errno == EINTR) continue;
        if (got <= 0) {
            if (got < 0) std::perror("read_noshort");
            break;
        }
        done += static_cast<std::size_t>(got);
    }
    return done;
}

std::size_t write_noshort(int fd, const void *src, std::size_t size)
{
    std::size_t done = 0;
    while (done < size) {
        const ssize_t put = ::write(fd, static_cast<const u8 *>(src) + done, size - done);
        if (put < 0 && errno == EINTR) continue;
        if (put <= 0) {
            std::perror("write_noshort");
            break;
        }
        done += static_cast<std::size_t>(put);
    }
    return done;
}
