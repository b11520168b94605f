// GGUF container reader: header, key-values, tensor infos, and zero-copy access to tensor bytes
// through a read-only mapping of the file.
//
// Follows the reader in /root/reference/fs/gguf/gguf.go (Open :54-110, readTensor :112-145,
// readKeyValue :147-201, readString/readArray :208-301, KeyValue lookup :332-351, TensorReader
// :390-430) and the size rule of /root/reference/fs/gguf/tensor.go:47-76:
//   "GGUF" | u32 version (>= 2) | u64 tensor count | u64 key-value count
//   key-values:   string key | u32 type | value        (string = u64 length + bytes;
//                                                       array = u32 element type | u64 count | elements)
//   tensor infos: string name | u32 n_dims (<= 4) | u64 dims[n_dims] | u32 type | u64 offset
//   padding to general.alignment (default 32), then the tensor data; a tensor's bytes start at
//   data_offset + its offset.
// Limits as in the reference: strings <= 16 MiB, arrays <= 64 Mi elements.  The reference parses
// lazily and reports errors from later calls; this reader parses everything in open() -- same
// values, errors surface earlier.  Plain host C++: no GPU involved.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace miqmm {

enum GgufValueType : uint32_t {
    GGUF_U8 = 0, GGUF_I8, GGUF_U16, GGUF_I16, GGUF_U32, GGUF_I32, GGUF_F32, GGUF_BOOL, GGUF_STRING, GGUF_ARRAY,
    GGUF_U64, GGUF_I64, GGUF_F64
};

struct GgufValue {
    uint32_t type = 0;       // GgufValueType
    uint32_t elem_type = 0;  // for arrays
    uint64_t count = 0;      // array length
    const uint8_t *data = nullptr;  // scalar: the value; string: the bytes; fixed-size array: the elements
    uint64_t len = 0;               // string length
    std::vector<std::pair<const uint8_t *, uint64_t>> strings;  // string arrays
};

struct GgufKV {
    std::string key;
    GgufValue value;
};

struct GgufTensor {
    std::string name;
    uint32_t type = 0;
    uint32_t n_dims = 0;
    uint64_t dims[4] = {1, 1, 1, 1};
    uint64_t offset = 0;  // relative to the data section
    int64_t nbytes = 0;
};

// elements per block and bytes per block by tensor type id (/root/reference/fs/gguf/tensor.go:152-239)
inline bool gguf_type_geometry(uint32_t type, int64_t &block, int64_t &bytes) {
    switch (type) {
    case 0: block = 1; bytes = 4; return true;        // F32
    case 1: block = 1; bytes = 2; return true;        // F16
    case 2: block = 32; bytes = 18; return true;      // Q4_0
    case 3: block = 32; bytes = 20; return true;      // Q4_1
    case 6: block = 32; bytes = 22; return true;      // Q5_0
    case 7: block = 32; bytes = 24; return true;      // Q5_1
    case 8: block = 32; bytes = 34; return true;      // Q8_0
    case 9: block = 32; bytes = 36; return true;      // Q8_1
    case 10: block = 256; bytes = 84; return true;    // Q2_K
    case 11: block = 256; bytes = 110; return true;   // Q3_K
    case 12: block = 256; bytes = 144; return true;   // Q4_K
    case 13: block = 256; bytes = 176; return true;   // Q5_K
    case 14: block = 256; bytes = 210; return true;   // Q6_K
    case 15: block = 256; bytes = 292; return true;   // Q8_K
    case 16: block = 256; bytes = 66; return true;    // IQ2_XXS
    case 17: block = 256; bytes = 74; return true;    // IQ2_XS
    case 18: block = 256; bytes = 98; return true;    // IQ3_XXS
    case 19: block = 256; bytes = 50; return true;    // IQ1_S
    case 20: block = 32; bytes = 18; return true;     // IQ4_NL
    case 21: block = 256; bytes = 110; return true;   // IQ3_S
    case 22: block = 256; bytes = 82; return true;    // IQ2_S
    case 23: block = 256; bytes = 136; return true;   // IQ4_XS
    case 24: block = 1; bytes = 1; return true;       // I8
    case 25: block = 1; bytes = 2; return true;       // I16
    case 26: block = 1; bytes = 4; return true;       // I32
    case 27: block = 1; bytes = 8; return true;       // I64
    case 28: block = 1; bytes = 8; return true;       // F64
    case 29: block = 256; bytes = 56; return true;    // IQ1_M
    case 30: block = 1; bytes = 2; return true;       // BF16
    case 39: block = 32; bytes = 17; return true;     // MXFP4
    case 40: block = 64; bytes = 36; return true;     // NVFP4
    case 41: block = 128; bytes = 18; return true;    // Q1_0
    default: return false;
    }
}

class GgufFile {
public:
    static constexpr uint64_t MAX_STRING = 16ull << 20, MAX_ARRAY = 64ull << 20;

    ~GgufFile() { close(); }

    // returns an empty string on success, else what went wrong
    std::string open(const char *path) {
        close();
        fd_ = ::open(path, O_RDONLY);
        if (fd_ < 0) return std::string("cannot open ") + path + ": " + strerror(errno);
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size < 24) return "file is shorter than a GGUF header";
        size_ = (uint64_t)st.st_size;
        void *m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (m == MAP_FAILED) return std::string("mmap failed: ") + strerror(errno);
        map_ = static_cast<const uint8_t *>(m);
        pos_ = 0;

        if (memcmp(map_, "GGUF", 4) != 0) return "unsupported file type (magic is not \"GGUF\")";
        pos_ = 4;
        if (!rd(version)) return "truncated header";
        if (version < 2) return "unsupported version " + std::to_string(version);
        uint64_t n_tensors, n_kv;
        if (!rd(n_tensors) || !rd(n_kv)) return "truncated header";
        // a key-value takes at least 12 bytes on disk, a tensor info at least 24
        if (n_kv > size_ / 12 || n_tensors > size_ / 24) return "item count exceeds what the file can hold";

        kvs.reserve(n_kv);
        for (uint64_t i = 0; i < n_kv; i++) {
            GgufKV kv;
            std::string e = read_kv(kv);
            if (!e.empty()) return "error reading GGUF item " + std::to_string(i) + ": " + e;
            kvs.push_back(std::move(kv));
        }
        tensors.reserve(n_tensors);
        for (uint64_t i = 0; i < n_tensors; i++) {
            GgufTensor t;
            std::string e = read_tensor(t);
            if (!e.empty()) return "error reading GGUF item " + std::to_string(i) + ": " + e;
            tensors.push_back(std::move(t));
        }
        int64_t al = 32;
        const int64_t idx = find_kv("general.alignment");
        if (idx >= 0) {
            // The writer stores it as u32 (/root/reference/fs/ggml/gguf.go:658); fs/gguf reads it with
            // Int() (gguf.go:89), fs/ggml with Uint(): accept either kind, 0 / absent means 32.
            int64_t v = as_int(kvs[idx].value);
            if (v == 0) v = (int64_t)as_uint(kvs[idx].value);
            if (v != 0) al = v;
        }
        if (al <= 0) return "unsupported alignment " + std::to_string(al);
        alignment = al;
        data_offset = pos_ + (alignment - pos_ % alignment) % alignment;
        for (const GgufTensor &t : tensors) {
            if (t.nbytes == 0) continue;
            if (t.offset > (uint64_t)INT64_MAX || data_offset + t.offset < data_offset)
                return "unsupported: tensor \"" + t.name + "\" offset overflows";
            if (data_offset > size_ || t.offset > size_ - data_offset || (uint64_t)t.nbytes > size_ - data_offset - t.offset)
                return "unsupported: tensor \"" + t.name + "\" offset+size exceeds file size";
        }
        return "";
    }

    void close() {
        if (map_) munmap(const_cast<uint8_t *>(map_), size_);
        if (fd_ >= 0) ::close(fd_);
        map_ = nullptr; fd_ = -1; size_ = 0;
        kvs.clear(); tensors.clear();
    }

    // keys outside "general." and "tokenizer." are looked up under the architecture's prefix
    int64_t find_kv(const std::string &key) const {
        std::string k = key;
        if (k.rfind("general.", 0) != 0 && k.rfind("tokenizer.", 0) != 0) {
            const int64_t a = find_kv("general.architecture");
            k = (a >= 0 ? as_string(kvs[a].value) : std::string()) + "." + key;
        }
        for (size_t i = 0; i < kvs.size(); i++)
            if (kvs[i].key == k) return (int64_t)i;
        return -1;
    }
    int64_t find_tensor(const std::string &name) const {
        for (size_t i = 0; i < tensors.size(); i++)
            if (tensors[i].name == name) return (int64_t)i;
        return -1;
    }
    const uint8_t *tensor_data(const GgufTensor &t) const { return map_ + data_offset + t.offset; }

    // scalar conversions with the reference's rule: zero / empty unless the stored kind matches
    static int64_t as_int(const GgufValue &v) {
        switch (v.type) {
        case GGUF_I8: return *reinterpret_cast<const int8_t *>(v.data);
        case GGUF_I16: return ld<int16_t>(v.data);
        case GGUF_I32: return ld<int32_t>(v.data);
        case GGUF_I64: return ld<int64_t>(v.data);
        default: return 0;
        }
    }
    static uint64_t as_uint(const GgufValue &v) {
        switch (v.type) {
        case GGUF_U8: return *v.data;
        case GGUF_U16: return ld<uint16_t>(v.data);
        case GGUF_U32: return ld<uint32_t>(v.data);
        case GGUF_U64: return ld<uint64_t>(v.data);
        default: return 0;
        }
    }
    static double as_float(const GgufValue &v) {
        switch (v.type) {
        case GGUF_F32: return ld<float>(v.data);
        case GGUF_F64: return ld<double>(v.data);
        default: return 0.0;
        }
    }
    static bool as_bool(const GgufValue &v) { return v.type == GGUF_BOOL && *v.data != 0; }
    static std::string as_string(const GgufValue &v) {
        return v.type == GGUF_STRING ? std::string(reinterpret_cast<const char *>(v.data), v.len) : std::string();
    }
    static size_t elem_size(uint32_t t) {
        switch (t) {
        case GGUF_U8: case GGUF_I8: case GGUF_BOOL: return 1;
        case GGUF_U16: case GGUF_I16: return 2;
        case GGUF_U32: case GGUF_I32: case GGUF_F32: return 4;
        case GGUF_U64: case GGUF_I64: case GGUF_F64: return 8;
        default: return 0;
        }
    }
    // element i of an array as a scalar value of the element type
    static GgufValue array_elem(const GgufValue &v, uint64_t i) {
        GgufValue e;
        e.type = v.elem_type;
        if (v.elem_type == GGUF_STRING) { e.data = v.strings[i].first; e.len = v.strings[i].second; }
        else e.data = v.data + i * elem_size(v.elem_type);
        return e;
    }

    uint32_t version = 0;
    int64_t alignment = 32;
    uint64_t data_offset = 0;
    std::vector<GgufKV> kvs;
    std::vector<GgufTensor> tensors;

private:
    template <class T>
    static T ld(const uint8_t *p) { T v; memcpy(&v, p, sizeof(T)); return v; }  // files are little-endian, so is the host
    template <class T>
    bool rd(T &v) {
        if (size_ - pos_ < sizeof(T)) return false;
        memcpy(&v, map_ + pos_, sizeof(T));
        pos_ += sizeof(T);
        return true;
    }
    std::string read_string(const uint8_t *&p, uint64_t &n) {
        if (!rd(n)) return "unexpected end of file";
        if (n > MAX_STRING) return "string " + std::to_string(n) + " exceeds maximum " + std::to_string(MAX_STRING);
        if (size_ - pos_ < n) return "unexpected end of file";
        p = map_ + pos_;
        pos_ += n;
        return "";
    }
    std::string read_kv(GgufKV &kv) {
        const uint8_t *p; uint64_t n;
        std::string e = read_string(p, n);
        if (!e.empty()) return e;
        kv.key.assign(reinterpret_cast<const char *>(p), n);
        GgufValue &v = kv.value;
        if (!rd(v.type)) return "unexpected end of file";
        if (v.type == GGUF_STRING) return read_string(v.data, v.len);
        if (v.type == GGUF_ARRAY) {
            if (!rd(v.elem_type) || !rd(v.count)) return "unexpected end of file";
            if (v.count > MAX_ARRAY) return "array size " + std::to_string(v.count) + " exceeds maximum " + std::to_string(MAX_ARRAY);
            if (v.elem_type == GGUF_STRING) {
                if (v.count > (size_ - pos_) / 8) return "unexpected end of file";
                v.strings.resize(v.count);
                for (uint64_t i = 0; i < v.count; i++) {
                    e = read_string(v.strings[i].first, v.strings[i].second);
                    if (!e.empty()) return e;
                }
                return "";
            }
            const size_t es = elem_size(v.elem_type);
            if (es == 0) return "unsupported type " + std::to_string(v.elem_type);
            if (v.count > (size_ - pos_) / es) return "unexpected end of file";
            v.data = map_ + pos_;
            pos_ += v.count * es;
            return "";
        }
        const size_t es = elem_size(v.type);
        if (es == 0) return "unsupported type " + std::to_string(v.type);
        if (size_ - pos_ < es) return "unexpected end of file";
        v.data = map_ + pos_;
        pos_ += es;
        return "";
    }
    std::string read_tensor(GgufTensor &t) {
        const uint8_t *p; uint64_t n;
        std::string e = read_string(p, n);
        if (!e.empty()) return e;
        t.name.assign(reinterpret_cast<const char *>(p), n);
        if (!rd(t.n_dims)) return "unexpected end of file";
        if (t.n_dims > 4) return "unsupported tensor dimensions " + std::to_string(t.n_dims) + " exceeds maximum 4";
        for (uint32_t i = 0; i < t.n_dims; i++)
            if (!rd(t.dims[i])) return "unexpected end of file";
        if (!rd(t.type) || !rd(t.offset)) return "unexpected end of file";
        // number of bytes: values / block size * bytes per block; dimension 0 must hold whole blocks
        int64_t block, bytes;
        if (!gguf_type_geometry(t.type, block, bytes)) return "unsupported: tensor \"" + t.name + "\" size overflows";
        uint64_t values = 1;
        for (uint32_t i = 0; i < t.n_dims; i++) {
            if (t.dims[i] != 0 && values > (uint64_t)INT64_MAX / t.dims[i])
                return "unsupported: tensor \"" + t.name + "\" size overflows";
            values *= t.dims[i];
        }
        const uint64_t row = t.n_dims > 0 ? t.dims[0] : 1;
        if (row % (uint64_t)block != 0) return "unsupported: tensor \"" + t.name + "\" size overflows";
        const uint64_t blocks = values / (uint64_t)block;
        if (blocks > (uint64_t)INT64_MAX / (uint64_t)bytes) return "unsupported: tensor \"" + t.name + "\" size overflows";
        t.nbytes = (int64_t)(blocks * (uint64_t)bytes);
        return "";
    }

    int fd_ = -1;
    const uint8_t *map_ = nullptr;
    uint64_t size_ = 0, pos_ = 0;
};

}  // namespace miqmm
