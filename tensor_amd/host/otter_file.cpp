// Readers of the reference's model files; see otter_file.hpp for what mirrors what.
#include "otter_file.hpp"

#include <algorithm>
#include <cstring>
#include <fstream>

namespace otter {
namespace core {

namespace {

// The file format is defined by how the reference reads it (Tensor/Otter.cpp:12-75): whitespace-separated words,
// classified one at a time. An Item is what one classification step yields.
enum class Kind { KeyValue, BlockOpen, BlockClose, Comment, Stop };
struct Item {
    Kind kind;
    std::string key, value;
};

void strip(std::string& s, char c) { s.erase(std::remove(s.begin(), s.end(), c), s.end()); }

// the value after a colon: one word, or -- when the word opens a quotation that it does not close -- everything up
// to the closing quote (Tensor/Otter.cpp:12-23); the quotes themselves are dropped by the caller
std::string read_value(std::istream& in) {
    std::string v;
    in >> v;
    if (!v.empty() && v.front() == '"' && v.back() != '"') {
        std::string rest;
        std::getline(in, rest, '"');
        v += rest;
    }
    return v;
}

Item next_item(std::istream& in) {
    std::string word;
    in >> word;
    if (in.eof()) return {Kind::Stop, "", word};  // also when the last word ends the file without a newline
    std::string value;
    const size_t colon = word.find(':');
    if (colon != std::string::npos) {  // "key:" value | "key:value"
        value = colon + 1 == word.size() ? read_value(in) : word.substr(colon + 1);
        word.resize(colon);
    } else if (word.find('{') != std::string::npos) {  // "Name{"
        word.resize(word.find('{'));
        strip(word, ' ');
        return {Kind::BlockOpen, word, ""};
    } else if (word.find('}') != std::string::npos) {
        return {Kind::BlockClose, "", ""};
    } else if (word[0] == '#') {  // the rest of the line is a comment
        std::string rest;
        std::getline(in, rest, '\n');
        return {Kind::Comment, "", rest};
    } else if (word[0] == '$') {
        return {Kind::Stop, "", ""};
    } else {  // a bare word: what follows decides -- "{" opens a block, ":" (or ":value") makes it a key
        std::string second;
        in >> second;
        const size_t c2 = second.find(':');
        if (second.find('{') != std::string::npos) {
            strip(word, ' ');
            return {Kind::BlockOpen, word, ""};
        } else if (c2 == std::string::npos) {
            std::fprintf(stderr, "[Param] Syntax error didn't find ':' but get %s\n", second.c_str());
        } else {
            value = c2 + 1 == second.size() ? read_value(in) : second.substr(c2 + 1);
        }
    }
    strip(word, ' ');
    strip(value, '"');
    return {Kind::KeyValue, word, value};
}

// reads items up to the end of the enclosing block (or of the file) into `params` / `blocks`
template <typename AddParam, typename AddBlock>
void read_block_body(std::istream& in, AddParam add_param, AddBlock add_block) {
    for (Item it = next_item(in); it.kind != Kind::Stop && it.kind != Kind::BlockClose; it = next_item(in)) {
        if (it.kind == Kind::BlockOpen) {
            Otter inner(it.key);
            inner.parseBlueprint(in);
            add_block(std::move(inner));
        } else if (it.kind == Kind::KeyValue) {
            add_param(Param(it.key, it.value));
        }
    }
}

}  // namespace

bool Otter::parseBlueprint(std::istream& in) {
    read_block_body(
        in, [&](Param p) { params_.push_back(std::move(p)); }, [&](Otter o) { partners_.push_back(std::move(o)); });
    return true;
}

std::vector<Param> Otter::getParams() const {
    std::vector<Param> all(params_);
    for (const Otter& p : partners_) all.insert(all.end(), p.params_.begin(), p.params_.end());
    return all;
}

bool OtterLeader::readProject(const char* project_path) {
    std::ifstream f(project_path);
    if (!f.is_open()) {
        std::fprintf(stderr, "[OtterLeader] Open file fail!\n");
        return false;
    }
    return readProject(f);
}

// Tensor/Otter.cpp:203-236: the first item must be `name: ...`; then file-level parameters and layer blocks
bool OtterLeader::readProject(std::istream& in) {
    const Item title = next_item(in);
    if (title.kind == Kind::KeyValue && title.key == "name")
        project_name_ = title.value;
    else
        std::fprintf(stderr, "[OtterLeader] Syntax error!\n");
    read_block_body(
        in, [&](Param p) { params_.push_back(std::move(p)); }, [&](Otter o) { teams_.push_back(std::move(o)); });
    return true;
}

}  // namespace core

// ---------------------------------------------------------------------------------------------------
// weight streams
// ---------------------------------------------------------------------------------------------------
size_t DataReaderFromStdio::read(void* buf, size_t size) const { return std::fread(buf, 1, size, file_); }

size_t DataReaderFromStdio::remain() const {  // Tensor/DataReader.cpp:49-54 (the position is restored here)
    const long at = std::ftell(file_);
    std::fseek(file_, 0, SEEK_END);
    const long end = std::ftell(file_);
    std::fseek(file_, at, SEEK_SET);
    return (size_t)(end - at);
}

size_t DataReaderFromMemory::read(void* buf, size_t size) const {
    const size_t n = std::min(size, left_);
    std::memcpy(buf, p_, n);
    p_ += n;
    left_ -= n;
    return n;
}

static int64_t count_of(const std::vector<int64_t>& shape) {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
}

Tensor InitializerFromDataReader::load(const std::vector<int64_t>& shape, int) const {
    Tensor t = Tensor::empty(shape, ScalarType::Float);
    const size_t bytes = (size_t)count_of(shape) * sizeof(float);
    if (dr_.read(t.data_ptr(), bytes) != bytes) {
        std::fprintf(stderr, "Load weight fail!\n");
        return Tensor();
    }
    return t;
}

// IEEE binary16 -> binary32, every class of value (Tensor/TensorConversion.cpp, from_float16)
static float half_to_float(unsigned short h) {
    const unsigned sign = (unsigned)(h & 0x8000u) << 16;
    unsigned exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: renormalise
            int e = -1;
            do {
                ++e;
                man <<= 1;
            } while (!(man & 0x400u));
            bits = sign | (unsigned)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | man << 13;
    } else {
        bits = sign | (exp + 127 - 15) << 23 | man << 13;
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

static size_t align4(size_t n) { return (n + 3) & ~(size_t)3; }

Tensor InitializerNcnnFromDataReader::load(const std::vector<int64_t>& shape, int type) const {
    const size_t count = (size_t)count_of(shape);
    auto read_exact = [&](void* dst, size_t bytes, const char* what) {
        const size_t got = dr_.read(dst, bytes);
        if (got != bytes) std::fprintf(stderr, "ModelBin read %s failed %zu\n", what, got);
        return got == bytes;
    };
    if (type == 1) {  // a plain fp32 vector (bias, scales): no tag
        Tensor t = Tensor::empty(shape, ScalarType::Float);
        return read_exact(t.data_ptr(), count * sizeof(float), "weight_data") ? t : Tensor();
    }
    OTTER_CHECK(type == 0, "Unsupport ncnn weight type!");

    unsigned char tag_bytes[4];
    if (!read_exact(tag_bytes, 4, "flag_struct")) return Tensor();
    unsigned tag;
    std::memcpy(&tag, tag_bytes, 4);
    const unsigned byte_sum = tag_bytes[0] + tag_bytes[1] + tag_bytes[2] + tag_bytes[3];

    if (tag == 0x01306B47u) {  // fp16 payload
        std::vector<unsigned short> half(align4(count * 2) / 2);
        if (!read_exact(half.data(), align4(count * 2), "float16_weights")) return Tensor();
        Tensor t = Tensor::empty(shape, ScalarType::Float);
        float* p = t.data_ptr<float>();
        for (size_t i = 0; i < count; ++i) p[i] = half_to_float(half[i]);
        return t;
    }
    if (tag == 0x000D4B38u) {  // int8 payload -> a Byte tensor, which is what selects the int8 pipeline
        std::vector<signed char> q(align4(count));
        if (!read_exact(q.data(), q.size(), "int8_weights")) return Tensor();
        Tensor t = Tensor::empty(shape, ScalarType::Byte);
        std::memcpy(t.data_ptr(), q.data(), count);
        return t;
    }
    Tensor t = Tensor::empty(shape, ScalarType::Float);
    if (tag == 0x0002C056u) {  // raw fp32 with an explicit tag
        return read_exact(t.data_ptr(), count * sizeof(float), "weight_data") ? t : Tensor();
    }
    if (byte_sum != 0) {  // 256-entry table + one index byte per weight
        float table[256];
        if (!read_exact(table, sizeof(table), "quantization_value")) return Tensor();
        std::vector<unsigned char> index(align4(count));
        if (!read_exact(index.data(), index.size(), "index_array")) return Tensor();
        float* p = t.data_ptr<float>();
        for (size_t i = 0; i < count; ++i) p[i] = table[index[i]];
        return t;
    }
    // tag 0: raw fp32
    return read_exact(t.data_ptr(), count * sizeof(float), "weight_data") ? t : Tensor();
}

}  // namespace otter
