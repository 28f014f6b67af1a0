// ggml_file.cpp — GGJT parser and tokenizer.  Format and tokenizer rules follow the reference
// (ggml_file.cpp:17-122 the layout, :162-186 payload sizes, :188-335 the bigram-merge tokenizer); the code is
// written for a read-only mapping that is never trusted: every length is checked against the file size, and a
// malformed file leaves the object closed with a message instead of aborting the process.
#include "ggml_file.h"

#include <algorithm>
#include <cassert>
#include <cerrno>
#include <exception>
#include <cstring>
#include <fcntl.h>
#include <iostream>
#include <queue>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <utility>

#include "utils.h"

namespace {

constexpr u32 kMagicGGJT = 0x67676a74u;

// bounds-checked little-endian reader over the mapping
class Cursor {
public:
    Cursor(const u8 *base, std::size_t size) : base_(base), size_(size) {}
    [[nodiscard]] std::size_t at() const { return pos_; }
    [[nodiscard]] bool fits(std::size_t n) const { return n <= size_ - pos_; }
    void seek(std::size_t p) { pos_ = p; }
    bool u32_le(u32 &out)
    {
        if (!fits(4)) return false;
        std::memcpy(&out, base_ + pos_, 4);
        pos_ += 4;
        return true;
    }
    bool f32_le(float &out)
    {
        if (!fits(4)) return false;
        std::memcpy(&out, base_ + pos_, 4);
        pos_ += 4;
        return true;
    }
    bool bytes(std::string &out, std::size_t n)
    {
        if (!fits(n)) return false;
        out.assign(reinterpret_cast<const char *>(base_ + pos_), n);
        pos_ += n;
        return true;
    }

private:
    const u8 *base_;
    std::size_t size_, pos_ = 0;
};

}  // namespace

// ---------------------------------------------------------------------------------------------------------------
// descriptors
// ---------------------------------------------------------------------------------------------------------------
ggml_data_descriptor::ggml_data_descriptor(std::string name_, ggml_value_type ftype_, u32 model_version_, std::size_t offset_,
                                           u32 shape1_, u32 shape2_)
    : name(std::move(name_)), ftype(ftype_), model_version(model_version_), offset(offset_), shape1(shape1_), shape2(shape2_), size(0)
{
    size = size_in_file();
}

std::size_t ggml_data_descriptor::size_in_file() const
{
    const std::size_t n = static_cast<std::size_t>(shape1) * shape2;
    switch (ftype) {
    case ggml_value_type::f32: return n * 4;
    case ggml_value_type::f16: return n * 2;
    case ggml_value_type::q4_0: return n % 32 ? 0 : n / 32 * (model_version == 1 ? 20 : 18);  // f32 scale in v1, f16 after
    case ggml_value_type::q8_0: return n % 32 ? 0 : n / 32 * (model_version == 1 ? 36 : 34);
    default: return 0;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// open / parse
// ---------------------------------------------------------------------------------------------------------------
void ggml_file::fail(const std::string &why)
{
    problem = why;
    std::cerr << why << std::endl;
    if (mapping) munmap(mapping, mapping_size);
    mapping = nullptr;
    mapping_size = 0;
    tokens.clear();
    tables.clear();
    name_to_index.clear();
    piece_to_id.clear();
}

ggml_file::ggml_file(const char *filepath)
{
    const int fd = ::open(filepath, O_RDONLY);
    if (fd < 0) {
        fail(std::string("Cannot open ") + filepath + ": " + std::strerror(errno));
        return;
    }
    struct stat st{};
    if (fstat(fd, &st) < 0) {
        const int e = errno;
        ::close(fd);
        fail(std::string("Cannot stat ") + filepath + ": " + std::strerror(e));
        return;
    }
    mapping_size = static_cast<std::size_t>(st.st_size);
    void *m = mapping_size ? mmap(nullptr, mapping_size, PROT_READ, MAP_SHARED, fd, 0) : MAP_FAILED;
    const int map_errno = errno;
    ::close(fd);
    if (m == MAP_FAILED) {
        mapping_size = 0;
        fail(std::string("Cannot mmap ") + filepath + ": " + (st.st_size ? std::strerror(map_errno) : "empty file"));
        return;
    }
    mapping = static_cast<u8 *>(m);
    bool parsed = false;
    try {
        parsed = parse();
    } catch (const std::exception &e) {  // allocation failure on a hostile size field: the object ends closed, like any bad file
        problem.clear();
        fail(std::string("Malformed model file ") + filepath + ": " + e.what());
        return;
    }
    if (!parsed && problem.empty()) fail(std::string("Malformed model file ") + filepath);
}

ggml_file::~ggml_file()
{
    if (mapping) munmap(mapping, mapping_size);
}

bool ggml_file::parse()
{
    Cursor cur(mapping, mapping_size);
    u32 words[9];
    for (u32 &w : words)
        if (!cur.u32_le(w)) return fail("Model file shorter than its header"), false;
    header = {words[0], words[1], words[2], words[3], words[4], words[5], words[6], words[7], words[8]};
    if (header.magic != kMagicGGJT) return fail("Not a GGJT file (bad magic)"), false;
    if (!header.vocab_size || !header.n_heads || !header.n_layers || header.rot * header.n_heads != header.dim)
        return fail("Inconsistent model header"), false;

    // vocabulary: i32 length, bytes, f32 score.  A record is at least 8 bytes, so a count the rest of the file cannot
    // hold is refused before anything is sized by it.
    if (header.vocab_size > (mapping_size - cur.at()) / 8) return fail("Vocabulary size " + std::to_string(header.vocab_size) + " exceeds the file"), false;
    tokens.reserve(header.vocab_size);
    for (u32 id = 0; id < header.vocab_size; ++id) {
        u32 len;
        ggml_token tok;
        if (!cur.u32_le(len) || len > 0x7fffffffu || !cur.bytes(tok.text, len) || !cur.f32_le(tok.score))
            return fail("Truncated vocabulary"), false;
        piece_to_id.emplace(tok.text, id);  // keeps the first (lowest) id of a piece that occurs twice
        tokens.push_back(std::move(tok));
    }

    // tensor records until the cursor lands exactly on the end of the file
    while (cur.at() != mapping_size) {
        const std::size_t record_at = cur.at();
        u32 n_dims, name_len, type_id, ne0, ne1 = 0;
        if (!cur.u32_le(n_dims) || !cur.u32_le(name_len) || !cur.u32_le(type_id)) return fail("Truncated tensor record"), false;
        if (n_dims != 1 && n_dims != 2) return fail("Tensor with " + std::to_string(n_dims) + " dimensions"), false;
        if (!cur.u32_le(ne0) || (n_dims == 2 && !cur.u32_le(ne1))) return fail("Truncated tensor record"), false;
        std::string name;
        if (!cur.bytes(name, name_len) || name.find('\0') != std::string::npos) return fail("Bad tensor name"), false;
        if (!(type_id <= 3 || type_id == 8)) {
            const char *tn = ftype_name(static_cast<ggml_value_type>(type_id));
            return fail("Bad format for matrix in input file: unsupported type " + (tn ? std::string(tn) : std::to_string(type_id)) +
                        " for table " + name + " at offset " + std::to_string(record_at)), false;
        }
        // a matrix is stored as (ne0 = columns, ne1 = rows); a vector as (ne0 = length)
        const u32 shape1 = n_dims == 2 ? ne1 : ne0, shape2 = n_dims == 2 ? ne0 : 1;
        const std::size_t payload_at = (cur.at() + 31) & ~static_cast<std::size_t>(31);
        ggml_data_descriptor d(name, static_cast<ggml_value_type>(type_id), header.file_version, payload_at, shape1, shape2);
        if (d.size == 0 && static_cast<std::size_t>(shape1) * shape2 != 0)
            return fail("Tensor " + name + " has a type or shape this build cannot size"), false;
        if (payload_at > mapping_size || d.size > mapping_size - payload_at) return fail("Tensor " + name + " runs past the end of the file"), false;
        if (!name_to_index.emplace(name, static_cast<u32>(tables.size())).second) return fail("Tensor " + name + " appears twice"), false;
        tables.push_back(std::move(d));
        cur.seek(payload_at + tables.back().size);
    }

    const ggml_data_descriptor *w1 = find_buffer_descriptor("layers.0.feed_forward.w1");
    if (!w1) return fail("Model file has no layers.0.feed_forward.w1"), false;
    ff_size = w1->shape1;
    return true;
}

void ggml_file::print_info() const
{
    if (!is_open()) return;
    const char magic[5] = {static_cast<char>(header.magic), static_cast<char>(header.magic >> 8), static_cast<char>(header.magic >> 16),
                           static_cast<char>(header.magic >> 24), 0};
    std::cout << "       magic: " << magic << "\n"
              << "file_version: " << header.file_version << "\n"
              << "  vocab_size: " << header.vocab_size << "\n"
              << "         dim: " << header.dim << "\n"
              << " multiple_of: " << header.multiple_of << "\n"
              << "     n_heads: " << header.n_heads << "\n"
              << "    n_layers: " << header.n_layers << "\n"
              << "per head dim: " << header.rot << "\n"
              << "       ftype: " << header.ftype << "\n"
              << "fast_forward: " << ff_size << std::endl;
}

const ggml_data_descriptor *ggml_file::find_buffer_descriptor(const std::string &s) const
{
    auto it = name_to_index.find(s);
    if (it == name_to_index.end()) it = name_to_index.find(s + ".weight");
    return it == name_to_index.end() ? nullptr : &tables[it->second];
}

const ggml_data_descriptor &ggml_file::get_buffer_descriptor(const std::string &s) const
{
    const ggml_data_descriptor *d = find_buffer_descriptor(s);
    assert(d && "tensor not in the model file");
    static const ggml_data_descriptor none("", ggml_value_type::f32, 0, 0, 0, 0);
    return d ? *d : none;
}

// ---------------------------------------------------------------------------------------------------------------
// tokenizer
// ---------------------------------------------------------------------------------------------------------------
int ggml_file::token_id_of(const char *bytes, std::size_t n) const
{
    const auto it = piece_to_id.find(std::string(bytes, n));
    return it == piece_to_id.end() ? -1 : static_cast<int>(it->second);
}

namespace {

// a piece of the text still standing, linked to its neighbours
struct Piece {
    int prev, next;
    std::size_t at, len;  // byte range in the text; len 0 = swallowed by a merge
};

// a candidate merge of two adjacent pieces
struct Merge {
    int left, right;
    float score;
    std::size_t len;  // combined length when proposed: a later merge of either side makes it stale
};

// best score first; among equal scores the leftmost pair (ggml_file.cpp:204-208)
struct MergeOrder {
    bool operator()(const Merge &a, const Merge &b) const { return a.score < b.score || (a.score == b.score && a.left > b.left); }
};

std::size_t utf8_length(unsigned char first)
{
    static const std::size_t by_high_nibble[16] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 3, 4};
    return by_high_nibble[first >> 4];
}

}  // namespace

void ggml_file::tokenize(std::vector<u32> &output, const std::string &text, bool bos) const
{
    if (text.empty()) return;  // nothing at all, not even the BOS (ggml_file.cpp:251-253)
    if (bos) output.push_back(1);

    // one piece per UTF-8 character (a truncated last character keeps what is there)
    std::vector<Piece> pieces;
    for (std::size_t at = 0; at < text.size();) {
        const std::size_t len = std::min(text.size() - at, utf8_length(static_cast<unsigned char>(text[at])));
        const int idx = static_cast<int>(pieces.size());
        pieces.push_back({idx - 1, idx + 1, at, len});
        at += len;
    }
    pieces.back().next = -1;

    std::priority_queue<Merge, std::vector<Merge>, MergeOrder> candidates;
    auto propose = [&](int left, int right) {
        if (left < 0 || right < 0) return;
        const std::size_t len = pieces[left].len + pieces[right].len;
        const int id = token_id_of(text.data() + pieces[left].at, len);  // adjacent pieces are contiguous in the text
        if (id >= 0) candidates.push({left, right, tokens[id].score, len});
    };
    for (int i = 1; i < static_cast<int>(pieces.size()); ++i) propose(i - 1, i);

    while (!candidates.empty()) {
        const Merge m = candidates.top();
        candidates.pop();
        Piece &l = pieces[m.left], &r = pieces[m.right];
        if (l.len == 0 || r.len == 0 || l.len + r.len != m.len) continue;  // one side changed since the proposal
        l.len += r.len;
        r.len = 0;
        l.next = r.next;
        if (r.next >= 0) pieces[r.next].prev = m.left;
        propose(l.prev, m.left);
        propose(m.left, l.next);
    }

    for (int i = 0; i != -1; i = pieces[i].next) {
        const Piece &p = pieces[i];
        const int id = token_id_of(text.data() + p.at, p.len);
        if (id >= 0) {
            output.push_back(static_cast<u32>(id));
        } else {
            // no piece in the vocabulary: one byte token per byte, ids 3..258
            for (std::size_t j = 0; j < p.len; ++j) output.push_back(static_cast<unsigned char>(text[p.at + j]) + 3u);
        }
    }
}

std::string ggml_file::tokens_to_text(const u32 *ids, u32 count) const
{
    std::string out;
    for (u32 j = 0; j < count; ++j)
        if (ids[j] < tokens.size()) out += tokens[ids[j]].text;
    return out;
}
