// qm_safetensors.cpp — see qm_safetensors.hpp.
#include "qm_safetensors.hpp"

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <dirent.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace qm_engine {

namespace {

// Just enough JSON for a safetensors header: objects, arrays, strings, numbers, literals.
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool boolean = false;
    double number = 0.0;
    std::string text;
    std::vector<Json> items;
    std::vector<std::pair<std::string, Json>> members;

    const Json* member(const std::string& key) const {
        for (const auto& m : members)
            if (m.first == key) return &m.second;
        return nullptr;
    }
};

class JsonReader {
public:
    JsonReader(const char* begin, size_t size) : p_(begin), end_(begin + size) {}
    Json document() {
        Json v = value(0);
        blanks();
        if (p_ != end_) fail("text after the document");
        return v;
    }

private:
    const char* p_;
    const char* end_;

    [[noreturn]] void fail(const char* what) const { throw IoError(std::string("safetensors header: ") + what); }
    void blanks() {
        while (p_ != end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
    }
    bool take(char c) {
        blanks();
        if (p_ != end_ && *p_ == c) {
            ++p_;
            return true;
        }
        return false;
    }
    void expect(char c) {
        if (!take(c)) fail("unexpected character");
    }
    void word(const char* w) {
        const size_t n = std::strlen(w);
        if (static_cast<size_t>(end_ - p_) < n || std::memcmp(p_, w, n) != 0) fail("unknown literal");
        p_ += n;
    }
    static void utf8(std::string& out, unsigned cp) {
        if (cp < 0x80) {
            out.push_back(static_cast<char>(cp));
        } else if (cp < 0x800) {
            out.push_back(static_cast<char>(0xc0 | (cp >> 6)));
            out.push_back(static_cast<char>(0x80 | (cp & 0x3f)));
        } else if (cp < 0x10000) {
            out.push_back(static_cast<char>(0xe0 | (cp >> 12)));
            out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3f)));
            out.push_back(static_cast<char>(0x80 | (cp & 0x3f)));
        } else {
            out.push_back(static_cast<char>(0xf0 | (cp >> 18)));
            out.push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3f)));
            out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3f)));
            out.push_back(static_cast<char>(0x80 | (cp & 0x3f)));
        }
    }
    unsigned hex4() {
        if (end_ - p_ < 4) fail("short \\u escape");
        unsigned v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = *p_++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= static_cast<unsigned>(c - '0');
            else if (c >= 'a' && c <= 'f') v |= static_cast<unsigned>(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= static_cast<unsigned>(c - 'A' + 10);
            else fail("bad \\u escape");
        }
        return v;
    }
    std::string string() {
        blanks();
        if (p_ == end_ || *p_ != '"') fail("string expected");
        ++p_;
        std::string out;
        while (p_ != end_) {
            const char c = *p_++;
            if (c == '"') return out;
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (p_ == end_) break;
            const char e = *p_++;
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    unsigned cp = hex4();
                    if (cp >= 0xd800 && cp < 0xdc00 && end_ - p_ >= 6 && p_[0] == '\\' && p_[1] == 'u') {
                        p_ += 2;
                        const unsigned low = hex4();
                        cp = 0x10000 + ((cp - 0xd800) << 10) + (low - 0xdc00);
                    }
                    utf8(out, cp);
                    break;
                }
                default: fail("bad escape");
            }
        }
        fail("unterminated string");
    }
    Json value(int depth) {
        if (depth > 64) fail("nesting too deep");
        blanks();
        if (p_ == end_) fail("unexpected end");
        Json v;
        const char c = *p_;
        if (c == '{') {
            ++p_;
            v.kind = Json::Object;
            if (take('}')) return v;
            do {
                std::string key = string();
                expect(':');
                v.members.emplace_back(std::move(key), value(depth + 1));
            } while (take(','));
            expect('}');
        } else if (c == '[') {
            ++p_;
            v.kind = Json::Array;
            if (take(']')) return v;
            do {
                v.items.push_back(value(depth + 1));
            } while (take(','));
            expect(']');
        } else if (c == '"') {
            v.kind = Json::String;
            v.text = string();
        } else if (c == 't') {
            word("true");
            v.kind = Json::Bool;
            v.boolean = true;
        } else if (c == 'f') {
            word("false");
            v.kind = Json::Bool;
        } else if (c == 'n') {
            word("null");
        } else {
            const char* start = p_;
            while (p_ != end_ && (std::isdigit(static_cast<unsigned char>(*p_)) || *p_ == '-' || *p_ == '+' || *p_ == '.'
                                  || *p_ == 'e' || *p_ == 'E'))
                ++p_;
            if (p_ == start) fail("value expected");
            const std::string digits(start, p_);
            char* stop = nullptr;
            v.kind = Json::Number;
            v.number = std::strtod(digits.c_str(), &stop);
            if (stop == digits.c_str() || *stop != '\0') fail("bad number");
        }
        return v;
    }
};

uint64_t as_count(const Json& v, const char* what) {
    if (v.kind != Json::Number || v.number < 0.0 || v.number > 9.0e15 || v.number != static_cast<double>(static_cast<uint64_t>(v.number)))
        throw IoError(std::string("safetensors header: ") + what + " is not a non-negative integer");
    return static_cast<uint64_t>(v.number);
}

}  // namespace

size_t dtype_size(const std::string& d) {
    if (d == "F64" || d == "I64" || d == "U64") return 8;
    if (d == "F32" || d == "I32" || d == "U32") return 4;
    if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
    if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
    throw TensorError("unsupported dtype: " + d);
}

SafeFile::SafeFile(const std::string& path) {
    fd_ = ::open(path.c_str(), O_RDONLY);
    if (fd_ < 0) throw IoError("open failed: " + path);
    struct stat st {};
    if (::fstat(fd_, &st) != 0 || st.st_size < 0) {
        ::close(fd_);
        throw IoError("fstat failed: " + path);
    }
    size_ = static_cast<size_t>(st.st_size);
    if (size_ < 8) {
        ::close(fd_);
        throw IoError("short safetensors file: " + path);
    }
    void* m = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (m == MAP_FAILED) {
        ::close(fd_);
        throw IoError("mmap failed: " + path);
    }
    map_ = static_cast<uint8_t*>(m);
    try {
        uint64_t header_bytes = 0;
        for (int i = 7; i >= 0; --i) header_bytes = (header_bytes << 8) | map_[i];
        if (header_bytes == 0 || header_bytes > size_ - 8) throw IoError("bad safetensors header length: " + path);
        const Json root = JsonReader(reinterpret_cast<const char*>(map_ + 8), static_cast<size_t>(header_bytes)).document();
        if (root.kind != Json::Object) throw IoError("safetensors header is not an object: " + path);
        const uint64_t base = 8 + header_bytes;
        const uint64_t data_bytes = size_ - base;
        for (const auto& entry : root.members) {
            if (entry.first == "__metadata__") continue;
            const Json& meta = entry.second;
            const Json* dtype = meta.member("dtype");
            const Json* shape = meta.member("shape");
            const Json* offsets = meta.member("data_offsets");
            if (meta.kind != Json::Object || !dtype || dtype->kind != Json::String || !shape || shape->kind != Json::Array
                || !offsets || offsets->kind != Json::Array || offsets->items.size() != 2)
                throw IoError("malformed tensor entry: " + entry.first);
            TensorView t;
            t.name = entry.first;
            t.dtype = dtype->text;
            // every extent fits an int and the element count cannot wrap: a crafted shape must not multiply out to
            // the byte range of a smaller tensor
            uint64_t count = 1;
            for (const Json& d : shape->items) {
                const uint64_t extent = as_count(d, "an extent");
                if (extent > 0x7fffffffULL) throw TensorError("tensor extent beyond 2^31 - 1: " + t.name);
                if (extent != 0 && count > (1ULL << 62) / extent) throw TensorError("tensor element count overflows: " + t.name);
                count *= extent;
                t.shape.push_back(static_cast<int64_t>(extent));
            }
            const uint64_t begin = as_count(offsets->items[0], "an offset");
            const uint64_t end = as_count(offsets->items[1], "an offset");
            if (begin > end || end > data_bytes) throw IoError("tensor out of range: " + t.name);
            if (t.elements() * dtype_size(t.dtype) != end - begin) throw TensorError("tensor byte mismatch: " + t.name);
            t.data = map_ + base + begin;
            t.bytes = end - begin;
            if (!tensors_.emplace(t.name, t).second) throw TensorError("duplicate tensor " + t.name);
        }
    } catch (...) {
        ::munmap(map_, size_);
        ::close(fd_);
        throw;
    }
}

SafeFile::~SafeFile() {
    if (map_) ::munmap(map_, size_);
    if (fd_ >= 0) ::close(fd_);
}

ModelDirectory::ModelDirectory(const std::string& directory) {
    std::vector<std::string> paths;
    DIR* dir = ::opendir(directory.c_str());
    if (!dir) throw IoError("cannot list model directory: " + directory);
    while (const dirent* e = ::readdir(dir)) {
        const std::string name = e->d_name;
        const std::string ext = ".safetensors";
        if (name.size() > ext.size() && name.compare(name.size() - ext.size(), ext.size(), ext) == 0)
            paths.push_back(directory + "/" + name);
    }
    ::closedir(dir);
    std::sort(paths.begin(), paths.end());
    if (paths.empty()) throw IoError("no safetensors file in " + directory);
    for (const std::string& path : paths) {
        auto file = std::make_unique<SafeFile>(path);
        for (const auto& kv : file->tensors())
            if (!index_.emplace(kv.first, &kv.second).second) throw TensorError("duplicate tensor " + kv.first);
        files_.push_back(std::move(file));
    }
}

const TensorView* ModelDirectory::maybe_suffix(const std::string& suffix) const {
    const TensorView* found = nullptr;
    for (const auto& kv : index_) {
        const std::string& name = kv.first;
        if (name.size() >= suffix.size() && name.compare(name.size() - suffix.size(), suffix.size(), suffix) == 0) {
            if (found) throw TensorError("ambiguous tensor suffix: " + suffix);
            found = kv.second;
        }
    }
    return found;
}

const TensorView& ModelDirectory::suffix(const std::string& suffix) const {
    const TensorView* found = maybe_suffix(suffix);
    if (!found) throw TensorError("tensor suffix missing: " + suffix);
    return *found;
}

}  // namespace qm_engine
