// weights.hpp — model weights from safetensors files into backend tensors: the dense part of
// `load_model_weights_for_dtype` (catgrad-llm/src/utils/mod.rs:321-449) for the f32 target
// dtype.  Files are memory-mapped; every tensor goes to the backend straight from the
// mapping (the backend stages it through pinned memory), F32 as it is, BF16 as bit patterns
// that the backend widens on the device (utils/mod.rs:158-168 does it on the host), I64
// tensors are skipped (utils/mod.rs:348-351), anything else is an unsupported dtype
// (utils/mod.rs:441).  Keys are the tensor names, split at '.' by the reference
// (utils/mod.rs:399-401) and used whole by this driver's parameter map.
// Packed mixture-of-experts tensors (utils/mod.rs:354-397) are not handled: no graph of this
// driver uses them.
#pragma once
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstring>
#include <string>
#include <vector>

#include "interp.hpp"

namespace cgh {

struct WeightError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct TensorEntry {
    std::string name, dtype;
    Shape shape;
    uint64_t begin = 0, end = 0; // byte range inside the data section
};

// The JSON header of a safetensors file: {"name": {"dtype": "F32", "shape": [..], "data_offsets": [b, e]}, ...,
// "__metadata__": {...}}.  A small recursive-descent reader for exactly that grammar (objects, arrays,
// strings with escapes, non-negative integers); values it does not need are skipped.
class HeaderReader {
  public:
    HeaderReader(const char *p, size_t n) : p_(p), end_(p + n) {}

    std::vector<TensorEntry> parse() {
        std::vector<TensorEntry> out;
        ws();
        expect('{');
        ws();
        if (peek() == '}') return out;
        for (;;) {
            ws();
            std::string key = string();
            ws();
            expect(':');
            ws();
            if (key == "__metadata__") {
                skip_value();
            } else {
                TensorEntry e = entry();
                e.name = key;
                out.push_back(std::move(e));
            }
            ws();
            if (peek() == ',') {
                p_++;
                continue;
            }
            expect('}');
            break;
        }
        return out;
    }

  private:
    const char *p_, *end_;

    char peek() const {
        if (p_ >= end_) throw WeightError("safetensors header: unexpected end");
        return *p_;
    }
    void expect(char c) {
        if (peek() != c) throw WeightError(std::string("safetensors header: expected '") + c + "'");
        p_++;
    }
    void ws() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) p_++;
    }
    std::string string() {
        expect('"');
        std::string s;
        while (peek() != '"') {
            char c = *p_++;
            if (c == '\\') {
                char e = peek();
                p_++;
                switch (e) {
                case 'n': s += '\n'; break;
                case 't': s += '\t'; break;
                case 'r': s += '\r'; break;
                case 'b': s += '\b'; break;
                case 'f': s += '\f'; break;
                case 'u': // keep the escape as written: tensor names are ASCII in practice
                    s += "\\u";
                    break;
                default: s += e; break; // \" \\ \/
                }
            } else {
                s += c;
            }
        }
        p_++;
        return s;
    }
    uint64_t integer() {
        if (peek() < '0' || peek() > '9') throw WeightError("safetensors header: expected a non-negative integer");
        uint64_t v = 0;
        while (p_ < end_ && *p_ >= '0' && *p_ <= '9') {
            if (v > (UINT64_MAX - 9) / 10) throw WeightError("safetensors header: integer overflow");
            v = v * 10 + (uint64_t)(*p_++ - '0');
        }
        return v;
    }
    std::vector<uint64_t> int_array() {
        std::vector<uint64_t> v;
        expect('[');
        ws();
        if (peek() == ']') {
            p_++;
            return v;
        }
        for (;;) {
            ws();
            v.push_back(integer());
            ws();
            if (peek() == ',') {
                p_++;
                continue;
            }
            expect(']');
            return v;
        }
    }
    void skip_value() {
        ws();
        char c = peek();
        if (c == '"') {
            string();
        } else if (c == '{' || c == '[') {
            const char close = c == '{' ? '}' : ']';
            p_++;
            ws();
            if (peek() == close) {
                p_++;
                return;
            }
            for (;;) {
                ws();
                if (c == '{') {
                    string();
                    ws();
                    expect(':');
                }
                skip_value();
                ws();
                if (peek() == ',') {
                    p_++;
                    continue;
                }
                expect(close);
                return;
            }
        } else { // number / true / false / null
            while (p_ < end_ && *p_ != ',' && *p_ != '}' && *p_ != ']') p_++;
        }
    }
    TensorEntry entry() {
        TensorEntry e;
        bool have_dtype = false, have_shape = false, have_off = false;
        expect('{');
        for (;;) {
            ws();
            std::string k = string();
            ws();
            expect(':');
            ws();
            if (k == "dtype") {
                e.dtype = string();
                have_dtype = true;
            } else if (k == "shape") {
                for (uint64_t d : int_array()) e.shape.push_back((size_t)d);
                have_shape = true;
            } else if (k == "data_offsets") {
                std::vector<uint64_t> o = int_array();
                if (o.size() != 2) throw WeightError("safetensors header: data_offsets must have two entries");
                e.begin = o[0];
                e.end = o[1];
                have_off = true;
            } else {
                skip_value();
            }
            ws();
            if (peek() == ',') {
                p_++;
                continue;
            }
            expect('}');
            break;
        }
        if (!have_dtype || !have_shape || !have_off) throw WeightError("safetensors header: incomplete tensor entry");
        return e;
    }
};

class MappedFile {
  public:
    explicit MappedFile(const std::string &path) {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) throw WeightError("cannot open " + path);
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size < 8) {
            ::close(fd_);
            throw WeightError(path + ": not a safetensors file (shorter than its length field)");
        }
        size_ = (size_t)st.st_size;
        void *m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (m == MAP_FAILED) {
            ::close(fd_);
            throw WeightError("cannot map " + path);
        }
        data_ = static_cast<const unsigned char *>(m);
    }
    ~MappedFile() {
        if (data_) munmap(const_cast<unsigned char *>(data_), size_);
        if (fd_ >= 0) ::close(fd_);
    }
    MappedFile(const MappedFile &) = delete;
    MappedFile &operator=(const MappedFile &) = delete;
    const unsigned char *data() const { return data_; }
    size_t size() const { return size_; }

  private:
    int fd_ = -1;
    const unsigned char *data_ = nullptr;
    size_t size_ = 0;
};

struct LoadStats {
    size_t tensors = 0, params = 0, bytes = 0, skipped = 0;
    double seconds = 0;
};

inline LoadStats load_safetensors(Interpreter &i, const std::vector<std::string> &paths) {
    LoadStats st;
    auto t0 = std::chrono::steady_clock::now();
    for (const std::string &path : paths) {
        MappedFile f(path);
        uint64_t hlen = 0;
        for (int b = 7; b >= 0; b--) hlen = (hlen << 8) | f.data()[b]; // little-endian u64
        if (hlen > f.size() - 8) throw WeightError(path + ": header length exceeds the file");
        HeaderReader hr(reinterpret_cast<const char *>(f.data()) + 8, (size_t)hlen);
        const unsigned char *base = f.data() + 8 + hlen;
        const uint64_t avail = f.size() - 8 - hlen;
        for (const TensorEntry &e : hr.parse()) {
            if (e.dtype == "I64") { // e.g. num_batches_tracked: not a model weight
                st.skipped++;
                continue;
            }
            size_t n = 1;
            for (size_t d : e.shape) n *= d;
            const size_t width = e.dtype == "F32" ? 4 : e.dtype == "BF16" ? 2 : 0;
            if (!width) throw WeightError("UnsupportedDtype(" + e.dtype + ") for tensor " + e.name);
            if (e.end < e.begin || e.end > avail || e.end - e.begin != (uint64_t)n * width)
                throw WeightError(path + ": tensor " + e.name + " has a byte range that does not match its shape");
            const unsigned char *p = base + e.begin;
            if (width == 4)
                i.parameters[e.name] = i.backend.ndarray_from_vec_f32(reinterpret_cast<const float *>(p), n, e.shape);
            else
                i.parameters[e.name] = i.backend.from_bf16_bits(reinterpret_cast<const uint16_t *>(p), n, e.shape);
            st.tensors++;
            st.params += n;
            st.bytes += n * width;
        }
    }
    i.backend.sync(); // the mappings go away now; the staged copies have already left them
    st.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    return st;
}

} // namespace cgh
