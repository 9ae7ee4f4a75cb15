// GGUF (versions 2 and 3, little-endian) reader: header, metadata and tensor table, with the reference reader's
// acceptance rules (jitnn-gguf/src/main/java/ai/beestream/jitnn/gguf/GgufFile.java:100-175,428-572).  Host code only:
// the file is memory-mapped read-only and tensor bytes go from the mapping straight to HBM.
#pragma once
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

namespace jitnn {

struct GgmlTypeInfo {
    int id, block_values, block_bytes;
    const char *name;
};

// gguf/GgmlType.java:27-65
inline const GgmlTypeInfo *ggml_type(int id) {
    static const GgmlTypeInfo table[] = {
        {0, 1, 4, "F32"},     {1, 1, 2, "F16"},     {2, 32, 18, "Q4_0"},   {3, 32, 20, "Q4_1"},   {6, 32, 22, "Q5_0"},
        {7, 32, 24, "Q5_1"},  {8, 32, 34, "Q8_0"},  {9, 32, 36, "Q8_1"},   {10, 256, 84, "Q2_K"}, {11, 256, 110, "Q3_K"},
        {12, 256, 144, "Q4_K"}, {13, 256, 176, "Q5_K"}, {14, 256, 210, "Q6_K"}, {15, 256, 292, "Q8_K"}, {24, 1, 1, "I8"},
        {25, 1, 2, "I16"},    {26, 1, 4, "I32"},    {27, 1, 8, "I64"},     {28, 1, 8, "F64"},     {30, 1, 2, "BF16"}};
    for (const auto &t : table)
        if (t.id == id) return &t;
    return nullptr;
}

struct GgufTensor {
    std::string name;
    std::vector<long long> shape;  // outermost axis first (GGUF lists the innermost first)
    int type_id;
    long long offset;  // in the file
    long long bytes;   // -1 for a type this reader does not know
    long long numel;
};

struct GgufFile {
    std::string path;
    int fd = -1;
    const uint8_t *map = nullptr;
    long long size = 0;
    int version = 0, alignment = 32;
    long long data_offset = 0, kv_count = 0;
    std::string metadata_json;  // {"key": value, ...} in file order
    std::vector<GgufTensor> tensors;

    ~GgufFile() {
        if (map) munmap(const_cast<uint8_t *>(map), (size_t)size);
        if (fd >= 0) close(fd);
    }
    const GgufTensor *find(const char *name) const {
        for (const auto &t : tensors)
            if (t.name == name) return &t;
        return nullptr;
    }
};

// Sequential bounds-checked little-endian reads; any read past the end sets `truncated`.
struct GgufReader {
    const uint8_t *p;
    long long size, pos = 0;
    bool truncated = false;
    std::string err;
    int depth = 0;

    bool need(long long n) {
        if (n < 0 || pos + n > size) {
            truncated = true;
            return false;
        }
        return true;
    }
    template <class T>
    T get() {
        T v{};
        if (need((long long)sizeof(T))) {
            memcpy(&v, p + pos, sizeof(T));
            pos += (long long)sizeof(T);
        }
        return v;
    }
    // a uint64 count that must be plausible for the bytes left (GgufFile.java:463-469)
    bool count(const char *what, long long &n) {
        const uint64_t u = get<uint64_t>();
        if (truncated) return false;
        if (u > (uint64_t)(size - pos)) {
            err = std::string(what) + " " + std::to_string(u) + " exceeds the file";
            return false;
        }
        n = (long long)u;
        return true;
    }
    bool str(std::string &out) {
        long long n;
        if (!count("string length", n)) return false;
        if (!need(n)) return false;
        out.assign(reinterpret_cast<const char *>(p + pos), (size_t)n);
        pos += n;
        return true;
    }
};

inline void json_string(std::string &o, const std::string &s) {
    o += '"';
    for (unsigned char c : s) {
        if (c == '"' || c == '\\') {
            o += '\\';
            o += (char)c;
        } else if (c < 0x20) {
            char b[8];
            snprintf(b, sizeof b, "\\u%04x", c);
            o += b;
        } else {
            o += (char)c;  // UTF-8 passes through
        }
    }
    o += '"';
}

inline void json_double(std::string &o, double v, int digits) {
    char b[40];
    if (v != v || v - v != 0) {  // NaN or infinity: not JSON numbers
        o += "null";
        return;
    }
    snprintf(b, sizeof b, "%.*g", digits, v);
    o += b;
    if (!strpbrk(b, ".eEn")) o += ".0";  // keep floats distinguishable from integers
}

bool gguf_value(GgufReader &r, uint32_t type, std::string &o);

inline bool gguf_array(GgufReader &r, std::string &o) {
    if (++r.depth > 64) {  // GgufFile.java:498-506
        r.err = "arrays nested more than 64 deep";
        return false;
    }
    const uint32_t type = r.get<uint32_t>();
    long long n;
    if (!r.count("array length", n)) return false;
    if (n > 0x7fffffffLL) {
        r.err = "array of " + std::to_string(n) + " values";
        return false;
    }
    if (type > 12) {
        r.err = "unknown array element type " + std::to_string(type);
        return false;
    }
    o += '[';
    for (long long i = 0; i < n; ++i) {
        if (i) o += ',';
        if (!gguf_value(r, type, o)) return false;
    }
    o += ']';
    --r.depth;
    return true;
}

// metadata value of GGUF type `type` appended as JSON (GgufFile.java:479-496): integers of every width as integers
// (a uint64 above 2^63-1 reads as negative, as in the reference), float32/float64 as floats, bool, string, arrays
inline bool gguf_value(GgufReader &r, uint32_t type, std::string &o) {
    switch (type) {
    case 0: o += std::to_string((unsigned)r.get<uint8_t>()); break;
    case 1: o += std::to_string((int)r.get<int8_t>()); break;
    case 2: o += std::to_string((unsigned)r.get<uint16_t>()); break;
    case 3: o += std::to_string((int)r.get<int16_t>()); break;
    case 4: o += std::to_string((unsigned long long)r.get<uint32_t>()); break;
    case 5: o += std::to_string((int)r.get<int32_t>()); break;
    case 6: json_double(o, (double)r.get<float>(), 9); break;
    case 7: o += r.get<uint8_t>() != 0 ? "true" : "false"; break;
    case 8: {
        std::string s;
        if (!r.str(s)) return false;
        json_string(o, s);
        break;
    }
    case 9: return gguf_array(r, o);
    case 10:
    case 11: o += std::to_string((long long)r.get<int64_t>()); break;
    case 12: json_double(o, r.get<double>(), 17); break;
    default: r.err = "unknown metadata value type " + std::to_string(type) + " at byte " + std::to_string(r.pos - 4); return false;
    }
    return !r.truncated;
}

// Parses `f->map`; on failure returns false with the reason in `err` (the caller prefixes the path).
inline bool gguf_parse(GgufFile *f, std::string &err) {
    GgufReader r{f->map, f->size};
    if (f->size < 24 || r.get<uint32_t>() != 0x46554747u) {
        err = "not a GGUF file";
        return false;
    }
    const uint32_t version = r.get<uint32_t>();
    if (version != 2 && version != 3) {
        err = "GGUF version " + std::to_string(version) + " is not supported (2 and 3 are; big-endian files are not)";
        return false;
    }
    f->version = (int)version;
    long long tensor_count, kv_count;
    auto fail_r = [&]() {
        err = r.truncated && r.err.empty() ? "truncated GGUF file" : r.err;
        return false;
    };
    if (!r.count("tensor count", tensor_count) || !r.count("metadata count", kv_count)) return fail_r();
    f->kv_count = kv_count;
    std::string json = "{";
    long long alignment = 32;
    bool alignment_ok = true;
    for (long long i = 0; i < kv_count; ++i) {
        std::string key;
        if (!r.str(key)) return fail_r();
        const uint32_t type = r.get<uint32_t>();
        if (r.truncated) return fail_r();
        if (i) json += ',';
        json_string(json, key);
        json += ':';
        const size_t at = json.size();
        r.depth = 0;
        if (!gguf_value(r, type, json)) return fail_r();
        if (key == "general.alignment") {
            alignment_ok = type <= 5 || type == 10 || type == 11;  // a Number in the reference: any integer type
            if (alignment_ok) alignment = atoll(json.c_str() + at);
            else alignment_ok = (type == 6 || type == 12) && (alignment = (long long)atof(json.c_str() + at), true);
        }
    }
    json += '}';
    if (!alignment_ok || alignment <= 0 || alignment > 0x7fffffffLL || (alignment & (alignment - 1)) != 0) {
        err = "general.alignment is not a power of two";
        return false;
    }
    f->alignment = (int)alignment;
    f->metadata_json.swap(json);
    struct RawInfo {
        std::string name;
        std::vector<uint64_t> dims;
        uint32_t type;
        uint64_t offset;
    };
    std::vector<RawInfo> raw;
    for (long long i = 0; i < tensor_count; ++i) {
        RawInfo t;
        if (!r.str(t.name)) return fail_r();
        const uint32_t nd = r.get<uint32_t>();
        if (r.truncated) return fail_r();
        if (nd > 8) {
            err = "tensor " + t.name + " has " + std::to_string(nd) + " dimensions";
            return false;
        }
        for (uint32_t d = 0; d < nd; ++d) t.dims.push_back(r.get<uint64_t>());
        t.type = r.get<uint32_t>();
        t.offset = r.get<uint64_t>();
        if (r.truncated) return fail_r();
        raw.push_back(std::move(t));
    }
    const long long a = f->alignment;
    f->data_offset = (r.pos + a - 1) / a * a;
    for (auto &t : raw) {
        GgufTensor g;
        g.name = t.name;
        g.type_id = (int)t.type;
        if (t.offset > 0x7fffffffffffffffULL) {  // above 2^63: no such offset fits a file
            err = "tensor " + t.name + " has offset " + std::to_string(t.offset);
            return false;
        }
        long long numel = 1;
        for (size_t d = t.dims.size(); d-- > 0;) {  // innermost first in the file
            const uint64_t v = t.dims[d];
            if (v > 0x7fffffffffffffffULL) {
                err = "tensor " + t.name + " has dimension " + std::to_string(v);
                return false;
            }
            if (v != 0 && numel > 0x7fffffffffffffffLL / (long long)v) {
                err = "a tensor size or offset overflows";
                return false;
            }
            numel *= (long long)v;
            g.shape.push_back((long long)v);
        }
        g.numel = numel;
        if ((long long)t.offset > 0x7fffffffffffffffLL - f->data_offset) {
            err = "a tensor size or offset overflows";
            return false;
        }
        g.offset = f->data_offset + (long long)t.offset;
        const GgmlTypeInfo *ti = ggml_type(g.type_id);
        g.bytes = -1;
        if (ti) {
            if (numel % ti->block_values != 0) {
                err = std::string(ti->name) + ": " + std::to_string(numel) + " values is not a whole number of blocks of " +
                      std::to_string(ti->block_values);
                return false;
            }
            if (numel / ti->block_values > 0x7fffffffffffffffLL / ti->block_bytes) {
                err = "a tensor size or offset overflows";
                return false;
            }
            g.bytes = numel / ti->block_values * ti->block_bytes;
        }
        if ((long long)(t.offset % (uint64_t)a) != 0 || g.offset > f->size || (g.bytes >= 0 && g.bytes > f->size - g.offset)) {
            err = "tensor " + t.name + " lies outside the file or is not aligned";
            return false;
        }
        f->tensors.push_back(std::move(g));
    }
    return true;
}

// Opens and parses; returns nullptr with `err` set ("<path>: reason") on failure.
inline GgufFile *gguf_open(const char *path, std::string &err) {
    GgufFile *f = new GgufFile();
    f->path = path;
    f->fd = open(path, O_RDONLY);
    struct stat st;
    if (f->fd < 0 || fstat(f->fd, &st) != 0) {
        err = std::string(path) + ": cannot be opened";
        delete f;
        return nullptr;
    }
    f->size = (long long)st.st_size;
    if (f->size > 0) {
        void *m = mmap(nullptr, (size_t)f->size, PROT_READ, MAP_PRIVATE, f->fd, 0);
        if (m == MAP_FAILED) {
            err = std::string(path) + ": cannot be mapped";
            delete f;
            return nullptr;
        }
        f->map = static_cast<const uint8_t *>(m);
    }
    std::string why;
    if (!gguf_parse(f, why)) {
        err = std::string(path) + ": " + why;
        delete f;
        return nullptr;
    }
    return f;
}

}  // namespace jitnn
