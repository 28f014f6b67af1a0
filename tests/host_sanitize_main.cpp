// Driver for the sanitizer run of the host parser and tokenizer: opens every file named on the command line, and
// for files that parse walks the tensor table, tokenizes a few strings and converts them back.  Built by
// tests/test_host_sanitizers.py with -fsanitize=address,undefined; a finding aborts with a non-zero exit code.
#include <cstdio>
#include <string>
#include <vector>

#include "ggml_file.h"

int main(int argc, char **argv)
{
    unsigned long opened = 0, checksum = 0;
    for (int i = 1; i < argc; ++i) {
        ggml_file f(argv[i]);
        if (!f.is_open()) continue;
        ++opened;
        const unsigned char *base = static_cast<const unsigned char *>(f.data());
        for (const ggml_data_descriptor &d : f.get_tables()) {
            // first and last byte of every payload lie inside the mapping
            if (d.size) checksum += base[d.offset] + base[d.offset + d.size - 1];
            checksum += f.find_buffer_descriptor(d.name) != nullptr;
        }
        for (const char *text : {"", "hello world", " hello", "ab", "\xe6\x97\xa5\xe6\x9c\xac", "\xff\xfe", "aaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaa"}) {
            std::vector<u32> ids;
            f.tokenize(ids, text, true);
            checksum += f.tokens_to_text(ids.data(), static_cast<u32>(ids.size())).size();
        }
    }
    std::printf("opened %lu of %d, checksum %lu\n", opened, argc - 1, checksum);
    return 0;
}
