// .safetensors reader (behaviour of src/io/io_safetensors.cpp): header parsing with a small
// JSON reader of its own, bounds-checked data offsets, one read per tensor.
#include "axiom/io/safetensors.hpp"

#include <cstdint>
#include <cstring>
#include <fstream>

namespace axiom::io::safetensors {

namespace {

constexpr uint64_t MAX_HEADER_BYTES = 100ull * 1024 * 1024; // the format's own limit

DType parse_dtype(const std::string &s) { // src/io/io_safetensors.cpp:16-44
    static const std::pair<const char *, DType> table[] = {
        {"F16", DType::Float16}, {"BF16", DType::BFloat16}, {"F32", DType::Float32}, {"F64", DType::Float64}, {"I8", DType::Int8},
        {"I16", DType::Int16},   {"I32", DType::Int32},     {"I64", DType::Int64},   {"U8", DType::UInt8},    {"U16", DType::UInt16},
        {"U32", DType::UInt32},  {"U64", DType::UInt64},    {"BOOL", DType::Bool}};
    for (const auto &[name, dt] : table)
        if (s == name) return dt;
    throw FileFormatError("SafeTensors: unsupported dtype: " + s);
}

struct Entry {
    std::string name;
    DType dtype = DType::Float32;
    Shape shape;
    uint64_t begin = 0, end = 0; // byte range within the data section
};

// ---- the subset of JSON a safetensors header uses: objects, arrays, strings, non-negative
// integers; other values (inside __metadata__) are skipped structurally
class Json {
  public:
    explicit Json(const std::string &text) : s_(text) {}

    std::vector<Entry> header() {
        std::vector<Entry> out;
        ws();
        expect('{');
        ws();
        if (peek() == '}') return out;
        for (;;) {
            ws();
            const std::string key = string();
            ws();
            expect(':');
            ws();
            if (key == "__metadata__") skip_value();
            else out.push_back(entry(key));
            ws();
            if (peek() == ',') { ++i_; continue; }
            expect('}');
            return out;
        }
    }

  private:
    [[noreturn]] void fail(const std::string &what) const { throw FileFormatError("SafeTensors: malformed header (" + what + " at byte " + std::to_string(i_) + ")"); }
    char peek() const { return i_ < s_.size() ? s_[i_] : '\0'; }
    void ws() {
        while (i_ < s_.size() && (s_[i_] == ' ' || s_[i_] == '\n' || s_[i_] == '\t' || s_[i_] == '\r')) ++i_;
    }
    void expect(char c) {
        if (peek() != c) fail(std::string("expected '") + c + "'");
        ++i_;
    }
    std::string string() {
        expect('"');
        std::string out;
        while (i_ < s_.size() && s_[i_] != '"') {
            char c = s_[i_++];
            if (c == '\\') {
                if (i_ >= s_.size()) fail("unterminated escape");
                const char e = s_[i_++];
                switch (e) {
                case 'n': c = '\n'; break;
                case 't': c = '\t'; break;
                case 'r': c = '\r'; break;
                case 'b': c = '\b'; break;
                case 'f': c = '\f'; break;
                case 'u': { // keep the low byte of \uXXXX: tensor names are ASCII in practice
                    if (i_ + 4 > s_.size()) fail("short \\u escape");
                    c = static_cast<char>(std::stoul(s_.substr(i_, 4), nullptr, 16) & 0xFF);
                    i_ += 4;
                    break;
                }
                default: c = e; // \" \\ \/
                }
            }
            out.push_back(c);
        }
        expect('"');
        return out;
    }
    uint64_t integer() {
        if (peek() < '0' || peek() > '9') fail("expected a non-negative integer");
        uint64_t v = 0;
        while (peek() >= '0' && peek() <= '9') {
            if (v > (UINT64_MAX - 9) / 10) fail("integer overflow");
            v = v * 10 + static_cast<uint64_t>(s_[i_++] - '0');
        }
        return v;
    }
    std::vector<uint64_t> int_array() {
        std::vector<uint64_t> out;
        expect('[');
        ws();
        if (peek() == ']') { ++i_; return out; }
        for (;;) {
            ws();
            out.push_back(integer());
            ws();
            if (peek() == ',') { ++i_; continue; }
            expect(']');
            return out;
        }
    }
    // Nesting the reader follows before it gives up: __metadata__ values are flat in files written by the format's
    // own tools, and a header of nothing but opening brackets must not walk the stack down.
    static constexpr int MAX_DEPTH = 64;
    int depth_ = 0;
    void skip_value() {
        struct Level {
            int &d;
            explicit Level(int &depth) : d(depth) { ++d; }
            ~Level() { --d; }
        } level(depth_);
        if (depth_ > MAX_DEPTH) fail("values nested deeper than 64 levels");
        ws();
        const char c = peek();
        if (c == '"') { string(); return; }
        if (c == '{' || c == '[') {
            const char close = c == '{' ? '}' : ']';
            ++i_;
            ws();
            if (peek() == close) { ++i_; return; }
            for (;;) {
                ws();
                if (c == '{') { string(); ws(); expect(':'); }
                skip_value();
                ws();
                if (peek() == ',') { ++i_; continue; }
                expect(close);
                return;
            }
        }
        // number / true / false / null
        const size_t start = i_;
        while (i_ < s_.size() && s_[i_] != ',' && s_[i_] != '}' && s_[i_] != ']' && s_[i_] != ' ' && s_[i_] != '\n') ++i_;
        if (i_ == start) fail("expected a value");
    }
    Entry entry(const std::string &name) {
        Entry e;
        e.name = name;
        bool have_dtype = false, have_shape = false, have_offsets = false;
        expect('{');
        for (;;) {
            ws();
            const std::string key = string();
            ws();
            expect(':');
            ws();
            if (key == "dtype") { e.dtype = parse_dtype(string()); have_dtype = true; }
            else if (key == "shape") {
                for (uint64_t d : int_array()) e.shape.push_back(static_cast<size_t>(d));
                have_shape = true;
            } else if (key == "data_offsets") {
                const auto o = int_array();
                if (o.size() != 2 || o[1] < o[0]) fail("data_offsets of '" + name + "' must be [begin, end]");
                e.begin = o[0];
                e.end = o[1];
                have_offsets = true;
            } else skip_value();
            ws();
            if (peek() == ',') { ++i_; continue; }
            expect('}');
            break;
        }
        if (!have_dtype || !have_shape || !have_offsets) fail("tensor '" + name + "' lacks dtype, shape or data_offsets");
        return e;
    }

    const std::string &s_;
    size_t i_ = 0;
};

struct Opened {
    std::ifstream file;
    std::vector<Entry> entries;
    uint64_t data_start = 0, data_bytes = 0;
};

Opened open_file(const std::string &filename) { // src/io/io_safetensors.cpp:55-120
    Opened o;
    o.file.open(filename, std::ios::binary);
    if (!o.file.is_open()) throw SerializationError("SafeTensors: cannot open file: " + filename);
    o.file.seekg(0, std::ios::end);
    const uint64_t file_bytes = static_cast<uint64_t>(o.file.tellg());
    o.file.seekg(0);
    unsigned char len[8];
    if (file_bytes < 8 || !o.file.read(reinterpret_cast<char *>(len), 8)) throw FileFormatError("SafeTensors: failed to read header length");
    uint64_t n = 0;
    for (int i = 7; i >= 0; --i) n = (n << 8) | len[i];
    if (n > MAX_HEADER_BYTES || n > file_bytes - 8) throw FileFormatError("SafeTensors: header too large (" + std::to_string(n) + " bytes)");
    std::string header(n, '\0');
    if (n && !o.file.read(header.data(), static_cast<std::streamsize>(n))) throw FileFormatError("SafeTensors: failed to read header JSON");
    o.entries = Json(header).header();
    o.data_start = 8 + n;
    o.data_bytes = file_bytes - o.data_start;
    for (const Entry &e : o.entries) {
        // element count times element size, computed so that it cannot wrap around (shape [2^32, 2^32] is 0 elements
        // in 64-bit arithmetic and would pass for an empty byte range): no partial product may exceed the data section
        uint64_t want = dtype_size(e.dtype);
        bool zero = false;
        for (size_t d : e.shape) zero = zero || d == 0;
        if (zero) want = 0;
        else
            for (size_t d : e.shape) {
                if (want > o.data_bytes / d) throw FileFormatError("SafeTensors: tensor '" + e.name + "' has a shape larger than the file's data section");
                want *= d;
            }
        if (e.end - e.begin != want)
            throw FileFormatError("SafeTensors: tensor '" + e.name + "' spans " + std::to_string(e.end - e.begin) + " bytes, its shape and dtype need " +
                                  std::to_string(want));
        if (e.end > o.data_bytes) throw FileFormatError("SafeTensors: tensor '" + e.name + "' lies outside the file");
    }
    return o;
}

Tensor read_entry(Opened &o, const Entry &e, Device device) {
    Tensor t(e.shape, e.dtype, Device::CPU);
    const uint64_t bytes = e.end - e.begin;
    if (bytes) {
        o.file.seekg(static_cast<std::streamoff>(o.data_start + e.begin));
        if (!o.file.read(static_cast<char *>(t.data()), static_cast<std::streamsize>(bytes)))
            throw SerializationError("SafeTensors: failed to read tensor '" + e.name + "'");
    }
    return device == Device::GPU ? t.to(Device::GPU) : t;
}

} // namespace

bool is_safetensors_file(const std::string &filename) {
    static const std::string ext = ".safetensors";
    return filename.size() >= ext.size() && filename.compare(filename.size() - ext.size(), ext.size(), ext) == 0;
}

std::map<std::string, Tensor> load(const std::string &filename, Device device) {
    Opened o = open_file(filename);
    std::map<std::string, Tensor> out;
    for (const Entry &e : o.entries) out.emplace(e.name, read_entry(o, e, device));
    return out;
}

std::vector<std::string> list_tensors(const std::string &filename) {
    Opened o = open_file(filename);
    std::vector<std::string> names;
    for (const Entry &e : o.entries) names.push_back(e.name);
    return names;
}

Tensor load_tensor(const std::string &filename, const std::string &tensor_name, Device device) {
    Opened o = open_file(filename);
    for (const Entry &e : o.entries)
        if (e.name == tensor_name) return read_entry(o, e, device);
    throw SerializationError("SafeTensors: tensor '" + tensor_name + "' not found in " + filename);
}

} // namespace axiom::io::safetensors
