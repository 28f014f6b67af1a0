// ggml_file.h — GGJT model file: memory mapping, header / vocabulary / tensor table, SentencePiece-style
// tokenizer.  Same public interface as the reference's class (ggml_file.h:24-57); the members the reference
// reaches through `friend` declarations are plain const accessors here.
#pragma once

#include <cstddef>
#include <string>
#include <unordered_map>
#include <vector>

#include "types.h"

// the nine 32-bit words at the start of the file (ggml_file.h:12-22)
struct ggml_header {
    u32 magic, file_version, vocab_size, dim, multiple_of, n_heads, n_layers, rot, ftype;
};

struct ggml_token {
    std::string text;
    float score;
};

// one tensor record: where its payload sits in the mapping and what it holds (ggml_file.h:29-41)
class ggml_data_descriptor {
public:
    ggml_data_descriptor(std::string name, ggml_value_type ftype, u32 model_version, std::size_t offset, u32 shape1, u32 shape2);
    std::string name;
    ggml_value_type ftype;
    u32 model_version;
    std::size_t offset;
    u32 shape1;  // rows (ne1) of a matrix, length of a vector
    u32 shape2;  // columns (ne0) of a matrix, 1 for a vector
    std::size_t size;

    // payload bytes for this type / file version; 0 for types the path does not read (ggml_file.cpp:162-186)
    [[nodiscard]] std::size_t size_in_file() const;
};

class ggml_file {
public:
    explicit ggml_file(const char *filepath);
    ~ggml_file();
    ggml_file(const ggml_file &) = delete;
    ggml_file &operator=(const ggml_file &) = delete;

    void print_info() const;
    void tokenize(std::vector<u32> &output, const std::string &text, bool bos) const;
    [[nodiscard]] std::string tokens_to_text(const u32 *tokens, u32 count) const;
    // looks up `s`, then `s + ".weight"`; the name must exist (the reference asserts)
    [[nodiscard]] const ggml_data_descriptor &get_buffer_descriptor(const std::string &s) const;
    [[nodiscard]] const std::vector<ggml_token> &get_tokens() const { return tokens; }

    // ---- what the reference exposes to its friend classes -------------------------------------------------
    [[nodiscard]] bool is_open() const { return mapping != nullptr; }
    [[nodiscard]] const std::string &error() const { return problem; }   // why is_open() is false
    [[nodiscard]] const ggml_header &get_header() const { return header; }
    [[nodiscard]] u32 get_ff_size() const { return ff_size; }
    [[nodiscard]] const u8 *data() const { return mapping; }
    [[nodiscard]] std::size_t data_size() const { return mapping_size; }
    [[nodiscard]] const std::vector<ggml_data_descriptor> &get_tables() const { return tables; }
    [[nodiscard]] const ggml_data_descriptor *find_buffer_descriptor(const std::string &s) const;

private:
    bool parse();
    void fail(const std::string &why);
    [[nodiscard]] int token_id_of(const char *bytes, std::size_t n) const;

    u8 *mapping = nullptr;
    std::size_t mapping_size = 0;
    ggml_header header{};
    u32 ff_size = 0;
    std::vector<ggml_token> tokens;
    std::vector<ggml_data_descriptor> tables;
    std::unordered_map<std::string, u32> name_to_index;
    std::unordered_map<std::string, u32> piece_to_id;  // lowest id per distinct piece (first match wins)
    std::string problem;
};
