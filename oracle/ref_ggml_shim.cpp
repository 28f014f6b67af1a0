// ref_ggml_shim.cpp — C entry points over the REFERENCE's own ggml_file class, compiled from the sources
// where they lie (see Makefile target _ref).  TEST INFRASTRUCTURE ONLY: used to check the product's GGJT
// parser and tokenizer, and the files mkggml writes, against the reference implementation.
// Only the class's public interface is used (ggml_file.h:43-57).  Asserts stay enabled on purpose: the
// reference populates its name index inside an assert (ggml_file.cpp:120).
#include <cstring>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>
#include <sys/stat.h>

#include "ggml_file.h"

extern "C" {

void *ref_ggml_open(const char *path)
{
    struct stat st{};
    if (stat(path, &st) != 0 || st.st_size < 36)
        return nullptr;  // the reference would carry on with a null mapping
    return new ggml_file(path);
}

void ref_ggml_close(void *h) { delete static_cast<ggml_file *>(h); }

// print_info() is the only public view of the header: capture what it prints (ggml_file.cpp:132-145).
// out[0..8] = file_version, vocab_size, dim, multiple_of, n_heads, n_layers, rot, ftype, ff_size
int ref_ggml_header(void *h, unsigned *out)
{
    std::ostringstream cap;
    std::streambuf *old = std::cout.rdbuf(cap.rdbuf());
    static_cast<ggml_file *>(h)->print_info();
    std::cout.rdbuf(old);
    std::istringstream in(cap.str());
    std::string line;
    int k = 0;
    while (std::getline(in, line)) {
        auto colon = line.find(':');
        if (colon == std::string::npos)
            continue;
        if (line.find("magic") != std::string::npos)
            continue;
        if (k < 9)
            out[k++] = static_cast<unsigned>(std::stoul(line.substr(colon + 1)));
    }
    return k;
}

unsigned ref_ggml_vocab_size(void *h) { return static_cast<unsigned>(static_cast<ggml_file *>(h)->get_tokens().size()); }

// copies token text (not NUL terminated) and returns its length; score through *score
unsigned ref_ggml_token(void *h, unsigned id, char *buf, unsigned cap, float *score)
{
    auto const &t = static_cast<ggml_file *>(h)->get_tokens().at(id);
    unsigned n = static_cast<unsigned>(t.text.size());
    if (buf && cap)
        std::memcpy(buf, t.text.data(), n < cap ? n : cap);
    if (score)
        *score = t.score;
    return n;
}

// the name MUST exist (the reference asserts otherwise)
void ref_ggml_tensor(void *h, const char *name, unsigned *ftype, unsigned long long *offset, unsigned *shape1,
                     unsigned *shape2, unsigned long long *size)
{
    auto const &d = static_cast<ggml_file *>(h)->get_buffer_descriptor(name);
    *ftype = static_cast<unsigned>(d.ftype);
    *offset = d.offset;
    *shape1 = d.shape1;
    *shape2 = d.shape2;
    *size = d.size;
}

unsigned ref_ggml_tokenize(void *h, const char *text, unsigned text_len, int bos, unsigned *out, unsigned cap)
{
    std::vector<uint32_t> ids;
    static_cast<ggml_file *>(h)->tokenize(ids, std::string(text, text_len), bos != 0);
    for (size_t i = 0; i < ids.size() && i < cap; i++)
        out[i] = ids[i];
    return static_cast<unsigned>(ids.size());
}

unsigned ref_ggml_detokenize(void *h, const unsigned *ids, unsigned n, char *out, unsigned cap)
{
    std::string s = static_cast<ggml_file *>(h)->tokens_to_text(ids, n);
    unsigned len = static_cast<unsigned>(s.size());
    std::memcpy(out, s.data(), len < cap ? len : cap);
    return len;
}
}
