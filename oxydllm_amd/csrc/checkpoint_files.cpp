// On-disk formats that feed the quantized matmul library: GGUF and safetensors indexes over
// read-only memory maps, and the Hugging Face `quantization_config` check.
//
// reference: src/common/gguf_weights.rs (GgufWeights), src/common/weights.rs (ModelWeights,
// QuantScheme, try_get_quant), src/models/parsers/hf_parser.rs:451-585.  The GGUF container
// layout is the one candle-core 0.11's quantized::gguf_file reads (public ggml specification):
//   magic "GGUF", u32 version (1..3), tensor count, metadata count (u32 in v1, u64 after),
//   metadata pairs (string key, u32 type, value), tensor infos (string name, u32 n_dims,
//   dims, u32 ggml type, u64 offset), padding up to `general.alignment` (default 32), data.
// safetensors: u64 header length, JSON header {name: {dtype, shape, data_offsets}}, data.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cctype>
#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <map>
#include <new>
#include <exception>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "oxq_files.h"
#include "oxq_internal.hpp"

using oxq::fail;

namespace {

// ---------------------------------------------------------------------------------------------
// a small JSON document model (objects keep insertion order; numbers remember whether they were
// written as non-negative integers, which is what serde_json's as_u64 distinguishes)
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    double num = 0;
    bool is_u64 = false;
    uint64_t u64 = 0;
    bool is_i64 = false;
    int64_t i64 = 0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;

    const Json &at(const char *key) const {
        static const Json null_value;
        if (kind != Object) return null_value;
        // serde_json keeps the last of duplicate keys
        for (auto it = obj.rbegin(); it != obj.rend(); ++it)
            if (it->first == key) return it->second;
        return null_value;
    }
    bool is_null() const { return kind == Null; }
    const char *as_str(const char *dflt) const { return kind == String ? str.c_str() : dflt; }
};

struct JsonParser {
    const char *p, *end, *start;
    std::string err;
    int depth = 0;

    bool fail_at(const char *what) {
        if (err.empty()) err = std::string(what) + " at byte " + std::to_string(p - start);
        return false;
    }
    JsonParser(const char *s, size_t n) : p(s), end(s + n), start(s) {}

    void ws() {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
    }
    bool lit(const char *s) {
        size_t n = strlen(s);
        if (size_t(end - p) < n || memcmp(p, s, n) != 0) return fail_at("bad literal");
        p += n;
        return true;
    }
    static void utf8(std::string &o, uint32_t c) {
        if (c < 0x80) o += char(c);
        else if (c < 0x800) { o += char(0xC0 | (c >> 6)); o += char(0x80 | (c & 0x3F)); }
        else if (c < 0x10000) { o += char(0xE0 | (c >> 12)); o += char(0x80 | ((c >> 6) & 0x3F)); o += char(0x80 | (c & 0x3F)); }
        else { o += char(0xF0 | (c >> 18)); o += char(0x80 | ((c >> 12) & 0x3F)); o += char(0x80 | ((c >> 6) & 0x3F)); o += char(0x80 | (c & 0x3F)); }
    }
    bool hex4(uint32_t &v) {
        if (end - p < 4) return fail_at("short \\u escape");
        v = 0;
        for (int i = 0; i < 4; ++i) {
            char c = *p++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= c - '0';
            else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
            else return fail_at("bad \\u escape");
        }
        return true;
    }
    bool string(std::string &o) {
        if (p >= end || *p != '"') return fail_at("expected string");
        ++p;
        while (true) {
            if (p >= end) return fail_at("unterminated string");
            unsigned char c = *p++;
            if (c == '"') return true;
            if (c < 0x20) return fail_at("control character in string");
            if (c != '\\') { o += char(c); continue; }
            if (p >= end) return fail_at("unterminated escape");
            char e = *p++;
            switch (e) {
            case '"': o += '"'; break;
            case '\\': o += '\\'; break;
            case '/': o += '/'; break;
            case 'b': o += '\b'; break;
            case 'f': o += '\f'; break;
            case 'n': o += '\n'; break;
            case 'r': o += '\r'; break;
            case 't': o += '\t'; break;
            case 'u': {
                uint32_t c1;
                if (!hex4(c1)) return false;
                if (c1 >= 0xD800 && c1 < 0xDC00) {
                    uint32_t c2;
                    if (end - p < 2 || p[0] != '\\' || p[1] != 'u') return fail_at("lone surrogate");
                    p += 2;
                    if (!hex4(c2)) return false;
                    if (c2 < 0xDC00 || c2 > 0xDFFF) return fail_at("bad surrogate pair");
                    c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
                } else if (c1 >= 0xDC00 && c1 <= 0xDFFF) {
                    return fail_at("lone surrogate");
                }
                utf8(o, c1);
                break;
            }
            default: return fail_at("bad escape");
            }
        }
    }
    bool number(Json &v) {
        const char *s = p;
        bool neg = false, integral = true;
        if (p < end && *p == '-') { neg = true; ++p; }
        if (p >= end || !isdigit((unsigned char)*p)) return fail_at("bad number");
        if (*p == '0') ++p;
        else while (p < end && isdigit((unsigned char)*p)) ++p;
        if (p < end && *p == '.') {
            integral = false;
            ++p;
            if (p >= end || !isdigit((unsigned char)*p)) return fail_at("bad fraction");
            while (p < end && isdigit((unsigned char)*p)) ++p;
        }
        if (p < end && (*p == 'e' || *p == 'E')) {
            integral = false;
            ++p;
            if (p < end && (*p == '+' || *p == '-')) ++p;
            if (p >= end || !isdigit((unsigned char)*p)) return fail_at("bad exponent");
            while (p < end && isdigit((unsigned char)*p)) ++p;
        }
        std::string text(s, p);
        v.kind = Json::Number;
        v.num = strtod(text.c_str(), nullptr);
        if (integral) {
            errno = 0;
            if (!neg) {
                unsigned long long u = strtoull(text.c_str(), nullptr, 10);
                if (errno == 0) {
                    v.is_u64 = true;
                    v.u64 = u;
                    if (u <= uint64_t(INT64_MAX)) { v.is_i64 = true; v.i64 = int64_t(u); }
                }
            } else {
                long long i = strtoll(text.c_str(), nullptr, 10);
                if (errno == 0) {
                    v.is_i64 = true;
                    v.i64 = i;
                }
            }
        }
        return true;
    }
    bool value(Json &v) {
        if (++depth > 128) return fail_at("nesting too deep");
        ws();
        if (p >= end) return fail_at("unexpected end");
        bool ok = true;
        switch (*p) {
        case 'n': ok = lit("null"); v.kind = Json::Null; break;
        case 't': ok = lit("true"); v.kind = Json::Bool; v.b = true; break;
        case 'f': ok = lit("false"); v.kind = Json::Bool; v.b = false; break;
        case '"': v.kind = Json::String; ok = string(v.str); break;
        case '[': {
            ++p;
            v.kind = Json::Array;
            ws();
            if (p < end && *p == ']') { ++p; break; }
            while (ok) {
                v.arr.emplace_back();
                ok = value(v.arr.back());
                if (!ok) break;
                ws();
                if (p < end && *p == ',') { ++p; continue; }
                if (p < end && *p == ']') { ++p; break; }
                ok = fail_at("expected , or ]");
            }
            break;
        }
        case '{': {
            ++p;
            v.kind = Json::Object;
            ws();
            if (p < end && *p == '}') { ++p; break; }
            while (ok) {
                ws();
                std::string key;
                ok = string(key);
                if (!ok) break;
                ws();
                if (p >= end || *p != ':') { ok = fail_at("expected :"); break; }
                ++p;
                v.obj.emplace_back(std::move(key), Json());
                ok = value(v.obj.back().second);
                if (!ok) break;
                ws();
                if (p < end && *p == ',') { ++p; continue; }
                if (p < end && *p == '}') { ++p; break; }
                ok = fail_at("expected , or }");
            }
            break;
        }
        default: ok = number(v);
        }
        --depth;
        return ok;
    }
    bool document(Json &v) {
        if (!value(v)) return false;
        ws();
        if (p != end) return fail_at("trailing characters");
        return true;
    }
};

// ---------------------------------------------------------------------------------------------
struct Mapping {
    const uint8_t *base = nullptr;
    size_t len = 0;
    std::string path;
};

struct TensorEntry {
    std::string name;
    int file_dtype = 0;
    int ggml_type = -1;
    int gguf_quant = -1;
    std::vector<int64_t> dims;
    const uint8_t *data = nullptr;
    uint64_t nbytes = 0;
    int shard = 0;
};

struct MetaValue {
    int type = 0;
    uint64_t bits = 0;       // scalar payload, as stored (little endian, zero-extended)
    std::string str;
    int elem_type = 0;       // arrays
    uint64_t elem_count = 0;
    const uint8_t *elems = nullptr;  // fixed-size element arrays: the bytes in the mapping
};

}  // namespace

struct oxq_tensor_file {
    bool gguf = false;
    std::vector<Mapping> maps;
    std::map<std::string, TensorEntry> tensors;       // ordered by name
    std::vector<const TensorEntry *> order;           // filled after loading
    std::vector<std::pair<std::string, MetaValue>> meta;
    std::unordered_map<std::string, size_t> meta_index;

    ~oxq_tensor_file() {
        for (auto &m : maps)
            if (m.base && m.len) munmap(const_cast<uint8_t *>(m.base), m.len);
    }
};

namespace {

int map_file(const char *path, Mapping &m) {
    int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail(OXQ_ERR_IO, "cannot open %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) {
        int e = errno;
        close(fd);
        return fail(OXQ_ERR_IO, "cannot stat %s: %s", path, strerror(e));
    }
    m.len = size_t(st.st_size);
    m.path = path;
    if (m.len == 0) {
        close(fd);
        return fail(OXQ_ERR_FORMAT, "%s is empty", path);
    }
    void *base = mmap(nullptr, m.len, PROT_READ, MAP_PRIVATE, fd, 0);
    int e = errno;
    close(fd);
    if (base == MAP_FAILED) {
        m.len = 0;
        return fail(OXQ_ERR_IO, "cannot map %s: %s", path, strerror(e));
    }
    m.base = static_cast<const uint8_t *>(base);
    return OXQ_OK;
}

// ---- ggml type table: block elements, block bytes, file dtype, kernel format ---------------------
struct GgmlType {
    int id;
    const char *name;
    int64_t block_elems, block_bytes;
    int file_dtype;
    int gguf_quant;
};
const GgmlType kGgmlTypes[] = {
    {0, "F32", 1, 4, OXQ_FILE_F32, -1},
    {1, "F16", 1, 2, OXQ_FILE_F16, -1},
    {2, "Q4_0", 32, 18, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q4_0},
    {3, "Q4_1", 32, 20, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q4_1},
    {6, "Q5_0", 32, 22, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q5_0},
    {7, "Q5_1", 32, 24, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q5_1},
    {8, "Q8_0", 32, 34, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q8_0},
    {9, "Q8_1", 32, 36, OXQ_FILE_GGML_BLOCK, -1},
    {10, "Q2_K", 256, 84, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q2_K},
    {11, "Q3_K", 256, 110, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q3_K},
    {12, "Q4_K", 256, 144, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q4_K},
    {13, "Q5_K", 256, 176, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q5_K},
    {14, "Q6_K", 256, 210, OXQ_FILE_GGML_BLOCK, OXQ_GGUF_Q6_K},
    {15, "Q8_K", 256, 292, OXQ_FILE_GGML_BLOCK, -1},
    {30, "BF16", 1, 2, OXQ_FILE_BF16, -1},
};
const GgmlType *ggml_type(uint32_t id) {
    for (const auto &t : kGgmlTypes)
        if (uint32_t(t.id) == id) return &t;
    return nullptr;
}

// ---- bounds-checked little-endian reader -----------------------------------------------------
struct Reader {
    const uint8_t *base;
    size_t len, pos = 0;
    const char *path;
    bool ok = true;

    bool need(uint64_t n) {
        if (!ok || n > len - pos) { ok = false; return false; }
        return true;
    }
    template <typename T> T get() {
        T v{};
        if (!need(sizeof(T))) return v;
        memcpy(&v, base + pos, sizeof(T));
        pos += sizeof(T);
        return v;
    }
    // lengths and counts are u32 in version 1, u64 afterwards
    uint64_t count(uint32_t version) { return version == 1 ? get<uint32_t>() : get<uint64_t>(); }
    bool str(uint32_t version, std::string &o) {
        uint64_t n = count(version);
        if (!need(n)) return false;
        o.assign(reinterpret_cast<const char *>(base + pos), size_t(n));
        pos += size_t(n);
        // version 1 strings carry their terminator
        if (version == 1)
            while (!o.empty() && o.back() == '\0') o.pop_back();
        return true;
    }
};

int scalar_size(int type) {
    switch (type) {
    case OXQ_GGUF_U8: case OXQ_GGUF_I8: case OXQ_GGUF_BOOL: return 1;
    case OXQ_GGUF_U16: case OXQ_GGUF_I16: return 2;
    case OXQ_GGUF_U32: case OXQ_GGUF_I32: case OXQ_GGUF_F32: return 4;
    case OXQ_GGUF_U64: case OXQ_GGUF_I64: case OXQ_GGUF_F64: return 8;
    default: return 0;
    }
}

bool read_meta_value(Reader &r, uint32_t version, int type, MetaValue &v, int depth) {
    v.type = type;
    if (int sz = scalar_size(type)) {
        if (!r.need(sz)) return false;
        v.bits = 0;
        memcpy(&v.bits, r.base + r.pos, sz);
        r.pos += sz;
        return true;
    }
    if (type == OXQ_GGUF_STRING) return r.str(version, v.str);
    if (type == OXQ_GGUF_ARRAY) {
        if (depth > 4) { r.ok = false; return false; }
        v.elem_type = int(r.get<uint32_t>());
        v.elem_count = r.count(version);
        if (!r.ok) return false;
        if (int sz = scalar_size(v.elem_type)) {
            if (v.elem_count > (r.len - r.pos) / sz) { r.ok = false; return false; }
            v.elems = r.base + r.pos;
            r.pos += size_t(v.elem_count) * sz;
            return true;
        }
        if (v.elem_type == OXQ_GGUF_STRING || v.elem_type == OXQ_GGUF_ARRAY) {
            // variable-size elements (token tables, merges): walked to find their end, not kept
            v.elems = r.base + r.pos;
            for (uint64_t i = 0; i < v.elem_count && r.ok; ++i) {
                MetaValue skip;
                if (v.elem_type == OXQ_GGUF_STRING) {
                    uint64_t n = r.count(version);
                    if (r.need(n)) r.pos += size_t(n);
                } else {
                    read_meta_value(r, version, OXQ_GGUF_ARRAY, skip, depth + 1);
                }
            }
            return r.ok;
        }
    }
    r.ok = false;
    return false;
}

int load_gguf_shard(oxq_tensor_file *f, int shard) {
    const Mapping &m = f->maps[shard];
    const char *path = m.path.c_str();
    Reader r{m.base, m.len, 0, path};
    uint32_t magic = r.get<uint32_t>();
    if (!r.ok || magic != 0x46554747u)  // "GGUF"
        return fail(OXQ_ERR_FORMAT, "%s: not a GGUF file (magic 0x%08x)", path, magic);
    uint32_t version = r.get<uint32_t>();
    if (!r.ok || version < 1 || version > 3)
        return fail(OXQ_ERR_FORMAT, "%s: unsupported GGUF version %u", path, version);
    uint64_t n_tensors = r.count(version);
    uint64_t n_meta = r.count(version);
    if (!r.ok) return fail(OXQ_ERR_FORMAT, "%s: truncated GGUF header", path);
    // a tensor record is at least 24 bytes (name length, rank, type, offset), a metadata record at least 12
    if (n_tensors > m.len / 24 || n_meta > m.len / 12)
        return fail(OXQ_ERR_FORMAT, "%s: truncated or damaged GGUF header: %llu tensors and %llu metadata records cannot fit in %zu bytes", path,
                    (unsigned long long)n_tensors, (unsigned long long)n_meta, m.len);

    uint64_t alignment = 32;
    for (uint64_t i = 0; i < n_meta; ++i) {
        std::string key;
        MetaValue v;
        if (!r.str(version, key)) return fail(OXQ_ERR_FORMAT, "%s: truncated metadata key %llu", path, (unsigned long long)i);
        uint32_t type = r.get<uint32_t>();
        if (!r.ok || type > OXQ_GGUF_F64)
            return fail(OXQ_ERR_FORMAT, "%s: metadata '%s' has unknown value type %u", path, key.c_str(), type);
        if (!read_meta_value(r, version, int(type), v, 0))
            return fail(OXQ_ERR_FORMAT, "%s: truncated or malformed metadata value '%s'", path, key.c_str());
        if (key == "general.alignment") {
            // any unsigned or signed integer width is accepted for the alignment
            switch (v.type) {
            case OXQ_GGUF_U8: case OXQ_GGUF_U16: case OXQ_GGUF_U32: case OXQ_GGUF_U64:
            case OXQ_GGUF_I8: case OXQ_GGUF_I16: case OXQ_GGUF_I32: case OXQ_GGUF_I64:
                alignment = v.bits;
                break;
            default: break;
            }
            if (alignment == 0 || alignment > (1u << 30))
                return fail(OXQ_ERR_FORMAT, "%s: bad general.alignment %llu", path, (unsigned long long)alignment);
        }
        if (shard == 0) {  // metadata comes from the first shard
            auto it = f->meta_index.find(key);
            if (it != f->meta_index.end()) f->meta[it->second].second = std::move(v);
            else {
                f->meta_index[key] = f->meta.size();
                f->meta.emplace_back(std::move(key), std::move(v));
            }
        }
    }

    struct Info {
        std::string name;
        std::vector<int64_t> dims;
        const GgmlType *type;
        uint64_t offset;
    };
    std::vector<Info> infos;
    infos.reserve(size_t(std::min<uint64_t>(n_tensors, 1u << 20)));
    for (uint64_t i = 0; i < n_tensors; ++i) {
        Info info;
        if (!r.str(version, info.name)) return fail(OXQ_ERR_FORMAT, "%s: truncated tensor info %llu", path, (unsigned long long)i);
        uint32_t n_dims = r.get<uint32_t>();
        if (!r.ok || n_dims > OXQ_FILE_MAX_RANK)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has %u dimensions", path, info.name.c_str(), n_dims);
        info.dims.resize(n_dims);
        for (uint32_t d = 0; d < n_dims; ++d) {
            uint64_t v = r.count(version);
            if (v > uint64_t(INT64_MAX)) r.ok = false;
            info.dims[n_dims - 1 - d] = int64_t(v);  // stored innermost first
        }
        uint32_t type = r.get<uint32_t>();
        info.offset = r.get<uint64_t>();
        if (!r.ok) return fail(OXQ_ERR_FORMAT, "%s: truncated tensor info '%s'", path, info.name.c_str());
        info.type = ggml_type(type);
        if (!info.type)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has unknown ggml type %u", path, info.name.c_str(), type);
        infos.push_back(std::move(info));
    }
    uint64_t data_offset = (uint64_t(r.pos) + alignment - 1) / alignment * alignment;

    for (auto &info : infos) {
        // gguf_weights.rs:318-345: element count a multiple of the block size, slice inside the map
        uint64_t elems = 1;
        for (int64_t d : info.dims) {
            if (d != 0 && elems > UINT64_MAX / uint64_t(d))
                return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' element count overflows", path, info.name.c_str());
            elems *= uint64_t(d);
        }
        if (elems % uint64_t(info.type->block_elems) != 0)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s': tensor elements %llu not divisible by block size %lld", path,
                        info.name.c_str(), (unsigned long long)elems, (long long)info.type->block_elems);
        const uint64_t blocks = elems / uint64_t(info.type->block_elems);
        if (blocks > UINT64_MAX / uint64_t(info.type->block_bytes))  // one-element "blocks" (F32, F16 ...) can wrap
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s': byte count of %llu elements overflows", path,
                        info.name.c_str(), (unsigned long long)elems);
        uint64_t nbytes = blocks * uint64_t(info.type->block_bytes);
        uint64_t start = data_offset + info.offset;
        if (start < data_offset || start + nbytes < start)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s': tensor offset overflow", path, info.name.c_str());
        if (start + nbytes > m.len)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s': tensor slice (%llu..%llu) out of mmap bounds (%zu)", path,
                        info.name.c_str(), (unsigned long long)start, (unsigned long long)(start + nbytes), m.len);
        TensorEntry e;
        e.name = info.name;
        e.file_dtype = info.type->file_dtype;
        e.ggml_type = info.type->id;
        e.gguf_quant = info.type->gguf_quant;
        e.dims = std::move(info.dims);
        e.data = m.base + start;
        e.nbytes = nbytes;
        e.shard = shard;
        f->tensors[e.name] = std::move(e);
    }
    return OXQ_OK;
}

// ---- safetensors ---------------------------------------------------------------------------------
struct StDtype {
    const char *name;
    int file_dtype;
    int size;
};
const StDtype kStDtypes[] = {
    {"F32", OXQ_FILE_F32, 4},   {"F16", OXQ_FILE_F16, 2},   {"BF16", OXQ_FILE_BF16, 2}, {"F64", OXQ_FILE_F64, 8},
    {"U8", OXQ_FILE_U8, 1},     {"I8", OXQ_FILE_I8, 1},     {"U16", OXQ_FILE_U16, 2},   {"I16", OXQ_FILE_I16, 2},
    {"U32", OXQ_FILE_U32, 4},   {"I32", OXQ_FILE_I32, 4},   {"U64", OXQ_FILE_U64, 8},   {"I64", OXQ_FILE_I64, 8},
    {"BOOL", OXQ_FILE_BOOL, 1}, {"F8_E4M3", OXQ_FILE_F8_E4M3, 1}, {"F8_E5M2", OXQ_FILE_F8_E5M2, 1},
};

int load_safetensors_shard(oxq_tensor_file *f, int shard) {
    const Mapping &m = f->maps[shard];
    const char *path = m.path.c_str();
    if (m.len < 8) return fail(OXQ_ERR_FORMAT, "%s: too short for a safetensors header", path);
    uint64_t hlen;
    memcpy(&hlen, m.base, 8);
    if (hlen > m.len - 8 || hlen > (100u << 20))
        return fail(OXQ_ERR_FORMAT, "%s: safetensors header length %llu exceeds the file", path, (unsigned long long)hlen);
    Json doc;
    JsonParser jp(reinterpret_cast<const char *>(m.base + 8), size_t(hlen));
    if (!jp.document(doc) || doc.kind != Json::Object)
        return fail(OXQ_ERR_FORMAT, "%s: safetensors header is not a JSON object (%s)", path, jp.err.c_str());
    const uint8_t *data = m.base + 8 + hlen;
    uint64_t data_len = m.len - 8 - hlen;
    for (const auto &kv : doc.obj) {
        if (kv.first == "__metadata__") continue;
        const Json &t = kv.second;
        const Json &dt = t.at("dtype"), &shape = t.at("shape"), &offs = t.at("data_offsets");
        if (dt.kind != Json::String || shape.kind != Json::Array || offs.kind != Json::Array || offs.arr.size() != 2 ||
            !offs.arr[0].is_u64 || !offs.arr[1].is_u64)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has a malformed header entry", path, kv.first.c_str());
        const StDtype *sd = nullptr;
        for (const auto &d : kStDtypes)
            if (dt.str == d.name) sd = &d;
        if (!sd) return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has unknown dtype '%s'", path, kv.first.c_str(), dt.str.c_str());
        if (shape.arr.size() > OXQ_FILE_MAX_RANK)
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has %zu dimensions", path, kv.first.c_str(), shape.arr.size());
        TensorEntry e;
        uint64_t elems = 1;
        for (const Json &d : shape.arr) {
            if (!d.is_u64 || d.u64 > uint64_t(INT64_MAX) || (d.u64 != 0 && elems > UINT64_MAX / d.u64))
                return fail(OXQ_ERR_FORMAT, "%s: tensor '%s' has a bad shape", path, kv.first.c_str());
            elems *= d.u64;
            e.dims.push_back(int64_t(d.u64));
        }
        uint64_t b = offs.arr[0].u64, en = offs.arr[1].u64;
        if (b > en || en > data_len || elems > UINT64_MAX / sd->size || en - b != elems * uint64_t(sd->size))
            return fail(OXQ_ERR_FORMAT, "%s: tensor '%s': data_offsets [%llu, %llu) do not match shape and dtype", path,
                        kv.first.c_str(), (unsigned long long)b, (unsigned long long)en);
        e.name = kv.first;
        e.file_dtype = sd->file_dtype;
        e.data = data + b;
        e.nbytes = en - b;
        e.shard = shard;
        f->tensors[e.name] = std::move(e);
    }
    return OXQ_OK;
}

int open_files(const char *op, const char *const *paths, int n_paths, bool gguf, oxq_tensor_file **out) {
    if (!out) return fail(OXQ_ERR_ARG, "%s: out is NULL", op);
    *out = nullptr;
    if (!paths || n_paths < 1) return fail(OXQ_ERR_ARG, "%s: paths must be non-empty", op);
    auto *f = new oxq_tensor_file;
    f->gguf = gguf;
    f->maps.resize(n_paths);
    for (int i = 0; i < n_paths; ++i) {
        if (!paths[i]) {
            delete f;
            return fail(OXQ_ERR_ARG, "%s: path %d is NULL", op, i);
        }
        int st = map_file(paths[i], f->maps[i]);
        if (st == OXQ_OK) st = gguf ? load_gguf_shard(f, i) : load_safetensors_shard(f, i);
        if (st != OXQ_OK) {
            delete f;
            return st;
        }
    }
    f->order.reserve(f->tensors.size());
    for (const auto &kv : f->tensors) f->order.push_back(&kv.second);
    *out = f;
    return OXQ_OK;
}

void fill(const TensorEntry &e, oxq_file_tensor *out) {
    memset(out, 0, sizeof *out);
    out->name = e.name.c_str();
    out->file_dtype = e.file_dtype;
    out->ggml_type = e.ggml_type;
    out->gguf_quant = e.gguf_quant;
    out->rank = int32_t(e.dims.size());
    for (size_t i = 0; i < e.dims.size(); ++i) out->dims[i] = e.dims[i];
    out->data = e.data;
    out->nbytes = e.nbytes;
    out->shard = e.shard;
}

const TensorEntry *exact(const oxq_tensor_file *f, const std::string &name) {
    auto it = f->tensors.find(name);
    return it == f->tensors.end() ? nullptr : &it->second;
}

// weights.rs:452-503 resolve_name
const TensorEntry *resolve(const oxq_tensor_file *f, const std::string &name) {
    if (const TensorEntry *e = exact(f, name)) return e;
    if (f->gguf) return nullptr;
    if (name.rfind("model.", 0) == 0) {
        std::string rest = name.substr(6);
        for (const char *prefix : {"model.language_model.", "model.language_model.model.", "language_model.",
                                   "language_model.model.", "model.model."})
            if (const TensorEntry *e = exact(f, prefix + rest)) return e;
    }
    if (name == "lm_head.weight" || name == "lm_head.weight_scale_inv") {
        for (const char *prefix : {"model.", "model.language_model.", "model.language_model.model.", "language_model.",
                                   "language_model.model."})
            if (const TensorEntry *e = exact(f, prefix + name)) return e;
    }
    return nullptr;
}

const MetaValue *meta(const oxq_tensor_file *f, const char *key) {
    auto it = f->meta_index.find(key);
    return it == f->meta_index.end() ? nullptr : &f->meta[it->second].second;
}

bool ieq(const char *a, const char *b) {
    for (; *a && *b; ++a, ++b)
        if (tolower((unsigned char)*a) != tolower((unsigned char)*b)) return false;
    return *a == *b;
}

// No exception may cross the C ABI (a Rust caller would abort or worse): every entry point below runs
// inside this guard, which turns std::bad_alloc and anything else thrown by the containers into a status.
template <typename F>
static int guarded(const char *op, F &&f) noexcept {
    try {
        return f();
    } catch (const std::bad_alloc &) {
        return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    } catch (const std::exception &e) {
        return fail(OXQ_ERR_RUNTIME, "%s: %s", op, e.what());
    } catch (...) {
        return fail(OXQ_ERR_RUNTIME, "%s: unexpected exception", op);
    }
}

}  // namespace

extern "C" {

int oxq_gguf_open(const char *const *paths, int n_paths, oxq_tensor_file **out) {
    return guarded("oxq_gguf_open", [&]() -> int {
        return open_files("oxq_gguf_open", paths, n_paths, true, out);
    });
}

int oxq_safetensors_open(const char *const *paths, int n_paths, oxq_tensor_file **out) {
    return guarded("oxq_safetensors_open", [&]() -> int {
        return open_files("oxq_safetensors_open", paths, n_paths, false, out);
    });
}

int oxq_tensor_file_close(oxq_tensor_file *f) {
    return guarded("oxq_tensor_file_close", [&]() -> int {
        delete f;
        return OXQ_OK;
    });
}

int64_t oxq_tensor_file_count(const oxq_tensor_file *f) { return f ? int64_t(f->order.size()) : 0; }

int oxq_tensor_file_at(const oxq_tensor_file *f, int64_t index, oxq_file_tensor *out) {
    return guarded("oxq_tensor_file_at", [&]() -> int {
        if (!f || !out) return fail(OXQ_ERR_ARG, "oxq_tensor_file_at: NULL argument");
        if (index < 0 || index >= int64_t(f->order.size()))
            return fail(OXQ_ERR_ARG, "oxq_tensor_file_at: index %lld out of [0, %zu)", (long long)index, f->order.size());
        fill(*f->order[size_t(index)], out);
        return OXQ_OK;
    });
}

int oxq_tensor_file_find(const oxq_tensor_file *f, const char *name, oxq_file_tensor *out, int *found) {
    return guarded("oxq_tensor_file_find", [&]() -> int {
        if (!f || !name || !out || !found) return fail(OXQ_ERR_ARG, "oxq_tensor_file_find: NULL argument");
        const TensorEntry *e = resolve(f, name);
        *found = e != nullptr;
        if (e) fill(*e, out);
        else memset(out, 0, sizeof *out);
        return OXQ_OK;
    });
}

uint64_t oxq_tensor_file_total_bytes(const oxq_tensor_file *f) {
    uint64_t total = 0;
    if (f)
        for (const TensorEntry *e : f->order) total += e->nbytes;
    return total;
}

int oxq_tensor_file_has_packed_quantized_weights(const oxq_tensor_file *f) {
    return guarded("oxq_tensor_file_has_packed_quantized_weights", [&]() -> int {
        if (!f) return 0;
        auto ends_with = [](const std::string &s, const char *suffix) {
            size_t n = strlen(suffix);
            return s.size() >= n && s.compare(s.size() - n, n, suffix) == 0;
        };
        for (const TensorEntry *e : f->order)
            if (ends_with(e->name, ".qweight") || ends_with(e->name, ".weight_packed")) return 1;
        return 0;
    });
}

int64_t oxq_gguf_metadata_count(const oxq_tensor_file *f) { return f ? int64_t(f->meta.size()) : 0; }

int oxq_gguf_metadata_at(const oxq_tensor_file *f, int64_t index, const char **key, int *value_type, int *elem_type,
                         uint64_t *elem_count) {
    return guarded("oxq_gguf_metadata_at", [&]() -> int {
        if (!f || !key || !value_type) return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_at: NULL argument");
        if (index < 0 || index >= int64_t(f->meta.size()))
            return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_at: index %lld out of [0, %zu)", (long long)index, f->meta.size());
        const auto &kv = f->meta[size_t(index)];
        *key = kv.first.c_str();
        *value_type = kv.second.type;
        if (elem_type) *elem_type = kv.second.type == OXQ_GGUF_ARRAY ? kv.second.elem_type : -1;
        if (elem_count) *elem_count = kv.second.type == OXQ_GGUF_ARRAY ? kv.second.elem_count : 0;
        return OXQ_OK;
    });
}

int oxq_gguf_metadata_u32(const oxq_tensor_file *f, const char *key, uint32_t *value, int *found) {
    return guarded("oxq_gguf_metadata_u32", [&]() -> int {
        if (!f || !key || !value || !found) return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_u32: NULL argument");
        const MetaValue *v = meta(f, key);
        *found = v && v->type == OXQ_GGUF_U32;
        if (*found) *value = uint32_t(v->bits);
        return OXQ_OK;
    });
}

int oxq_gguf_metadata_f32(const oxq_tensor_file *f, const char *key, float *value, int *found) {
    return guarded("oxq_gguf_metadata_f32", [&]() -> int {
        if (!f || !key || !value || !found) return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_f32: NULL argument");
        const MetaValue *v = meta(f, key);
        *found = v && v->type == OXQ_GGUF_F32;
        if (*found) {
            uint32_t b = uint32_t(v->bits);
            memcpy(value, &b, 4);
        }
        return OXQ_OK;
    });
}

int oxq_gguf_metadata_string(const oxq_tensor_file *f, const char *key, const char **value, uint64_t *len, int *found) {
    return guarded("oxq_gguf_metadata_string", [&]() -> int {
        if (!f || !key || !value || !found) return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_string: NULL argument");
        const MetaValue *v = meta(f, key);
        *found = v && v->type == OXQ_GGUF_STRING;
        if (*found) {
            *value = v->str.c_str();
            if (len) *len = v->str.size();
        }
        return OXQ_OK;
    });
}

int oxq_gguf_metadata_number(const oxq_tensor_file *f, const char *key, double *value, int *found) {
    return guarded("oxq_gguf_metadata_number", [&]() -> int {
        if (!f || !key || !value || !found) return fail(OXQ_ERR_ARG, "oxq_gguf_metadata_number: NULL argument");
        const MetaValue *v = meta(f, key);
        *found = 0;
        if (!v) return OXQ_OK;
        uint64_t b = v->bits;
        switch (v->type) {
        case OXQ_GGUF_U8: case OXQ_GGUF_U16: case OXQ_GGUF_U32: case OXQ_GGUF_U64: *value = double(b); break;
        case OXQ_GGUF_BOOL: *value = b ? 1.0 : 0.0; break;
        case OXQ_GGUF_I8: *value = double(int8_t(b)); break;
        case OXQ_GGUF_I16: *value = double(int16_t(b)); break;
        case OXQ_GGUF_I32: *value = double(int32_t(b)); break;
        case OXQ_GGUF_I64: *value = double(int64_t(b)); break;
        case OXQ_GGUF_F32: { uint32_t w = uint32_t(b); float x; memcpy(&x, &w, 4); *value = x; break; }
        case OXQ_GGUF_F64: { double x; memcpy(&x, &b, 8); *value = x; break; }
        default: return OXQ_OK;
        }
        *found = 1;
        return OXQ_OK;
    });
}

int oxq_gguf_architecture(const oxq_tensor_file *f, const char **value, uint64_t *len, int *found) {
    return guarded("oxq_gguf_architecture", [&]() -> int {
        return oxq_gguf_metadata_string(f, "general.architecture", value, len, found);
    });
}

int oxq_gguf_eos_token_ids(const oxq_tensor_file *f, uint32_t *ids, uint64_t cap, uint64_t *count) {
    return guarded("oxq_gguf_eos_token_ids", [&]() -> int {
        if (!f || !count || (!ids && cap)) return fail(OXQ_ERR_ARG, "oxq_gguf_eos_token_ids: NULL argument");
        std::vector<uint32_t> all;
        if (const MetaValue *v = meta(f, "tokenizer.ggml.eos_token_id"))
            if (v->type == OXQ_GGUF_U32) all.push_back(uint32_t(v->bits));
        if (const MetaValue *v = meta(f, "tokenizer.ggml.eos_token_ids"))
            if (v->type == OXQ_GGUF_ARRAY && v->elem_type == OXQ_GGUF_U32)
                for (uint64_t i = 0; i < v->elem_count; ++i) {
                    uint32_t id;
                    memcpy(&id, v->elems + 4 * i, 4);
                    if (std::find(all.begin(), all.end(), id) == all.end()) all.push_back(id);
                }
        *count = all.size();
        for (uint64_t i = 0; i < all.size() && i < cap; ++i) ids[i] = all[i];
        return OXQ_OK;
    });
}

int oxq_validate_quantization_config(const char *json, int whole_config, oxq_quant_scheme *out) {
    return guarded("oxq_validate_quantization_config", [&]() -> int {
        const char *op = "oxq_validate_quantization_config";
        if (!json || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
        out->kind = OXQ_SCHEME_NONE;
        out->bits = 0;
        out->sym = 0;
        Json doc;
        JsonParser jp(json, strlen(json));
        if (!jp.document(doc)) return fail(OXQ_ERR_FORMAT, "%s: %s", op, jp.err.c_str());
        const Json &v = whole_config ? doc.at("quantization_config") : doc;
        if (v.is_null()) return OXQ_OK;

        std::string method = v.at("quant_method").as_str("");
        for (char &c : method) c = char(tolower((unsigned char)c));
        const Json &bits = v.at("bits");
        const char *version = v.at("version").as_str("gemm");

        if (method == "awq") {
            if (!bits.is_u64)
                return fail(OXQ_ERR_UNSUPPORTED, "AWQ checkpoint missing required 'bits' field in quantization_config");
            uint32_t b = uint32_t(bits.u64);
            if (b != 4 && b != 8)
                return fail(OXQ_ERR_UNSUPPORTED, "AWQ checkpoint bits=%u not supported. Only 4 and 8 bits are recognised.", b);
            if (!ieq(version, "gemm"))
                return fail(OXQ_ERR_UNSUPPORTED, "AWQ version '%s' is not supported (only 'gemm' has a runtime path).", version);
            out->kind = OXQ_SCHEME_AWQ;
            out->bits = b;
            return OXQ_OK;
        }
        if (method == "fp8" || method == "mxfp4" || method.empty()) return OXQ_OK;
        if (method == "gptq") {
            if (!bits.is_u64)
                return fail(OXQ_ERR_UNSUPPORTED, "GPTQ checkpoint missing required 'bits' field in quantization_config");
            if (bits.u64 != 4 && bits.u64 != 8)
                return fail(OXQ_ERR_UNSUPPORTED, "GPTQ checkpoint bits=%llu not supported. Only 4 and 8 bits are recognised.",
                            (unsigned long long)bits.u64);
            const Json &sym = v.at("sym"), &desc = v.at("desc_act");
            bool s = sym.kind == Json::Bool ? sym.b : true;
            bool d = desc.kind == Json::Bool ? desc.b : false;
            if (d)
                return fail(OXQ_ERR_UNSUPPORTED, "GPTQ checkpoint has desc_act=true (act-order). Only desc_act=false "
                                                 "(sequential g_idx) is supported.");
            const char *fmt = v.at("checkpoint_format").as_str("gptq");
            if (!ieq(fmt, "gptq"))
                return fail(OXQ_ERR_UNSUPPORTED, "GPTQ checkpoint_format='%s' not supported (only the canonical 'gptq' format).",
                            fmt);
            out->kind = OXQ_SCHEME_GPTQ;
            out->bits = uint32_t(bits.u64);
            out->sym = s;
            return OXQ_OK;
        }
        if (method == "compressed-tensors") {
            const char *format = v.at("format").as_str("");
            if (strcmp(format, "pack-quantized") != 0)
                return fail(OXQ_ERR_UNSUPPORTED, "compressed-tensors format '%s' not supported (only 'pack-quantized')", format);
            const Json &groups = v.at("config_groups");
            size_t n_groups = 0;
            if (groups.kind == Json::Object) {
                // distinct keys (a JSON map keeps one value per key)
                std::vector<const std::string *> seen;
                for (const auto &kv : groups.obj) {
                    bool dup = false;
                    for (const std::string *s : seen) dup = dup || *s == kv.first;
                    if (!dup) seen.push_back(&kv.first);
                }
                n_groups = seen.size();
            }
            const Json &w = groups.at("group_0").at("weights");
            const Json &nb = w.at("num_bits"), &symm = w.at("symmetric");
            uint64_t num_bits = nb.is_u64 ? nb.u64 : 0;
            bool symmetric = symm.kind == Json::Bool ? symm.b : false;
            const char *wtype = w.at("type").as_str("");
            const char *strategy = w.at("strategy").as_str("");
            bool actorder = w.at("actorder").kind == Json::String;
            if (n_groups != 1 || num_bits != 4 || !symmetric || strcmp(wtype, "int") != 0 || strcmp(strategy, "group") != 0 ||
                actorder)
                return fail(OXQ_ERR_UNSUPPORTED,
                            "compressed-tensors config not supported: requires a single group with int4 symmetric "
                            "group-strategy weights, no actorder (got groups=%zu, bits=%llu, sym=%s, type='%s', strategy='%s', "
                            "actorder=%s)",
                            n_groups, (unsigned long long)num_bits, symmetric ? "true" : "false", wtype, strategy,
                            actorder ? "set" : "none");
            out->kind = OXQ_SCHEME_COMPRESSED_TENSORS4;
            out->bits = 4;
            out->sym = 1;
            return OXQ_OK;
        }
        return fail(OXQ_ERR_UNSUPPORTED,
                    "Unknown quantization method '%s' in quantization_config. Supported: awq (gemm, 4/8-bit), gptq (4/8-bit, "
                    "desc_act=false), compressed-tensors (pack-quantized int4), fp8, mxfp4.",
                    method.c_str());
    });
}

int oxq_safetensors_try_get_quant(const oxq_tensor_file *f, const oxq_quant_scheme *scheme, const char *prefix,
                                  oxq_file_tensor *qweight, oxq_file_tensor *qzeros, oxq_file_tensor *scales, int *found) {
    return guarded("oxq_safetensors_try_get_quant", [&]() -> int {
        if (!f || !scheme || !prefix || !qweight || !qzeros || !scales || !found)
            return fail(OXQ_ERR_ARG, "oxq_safetensors_try_get_quant: NULL argument");
        *found = 0;
        memset(qweight, 0, sizeof *qweight);
        memset(qzeros, 0, sizeof *qzeros);
        memset(scales, 0, sizeof *scales);
        std::string p(prefix);
        const TensorEntry *w = nullptr, *z = nullptr, *s = nullptr;
        switch (scheme->kind) {
        case OXQ_SCHEME_NONE: return OXQ_OK;
        case OXQ_SCHEME_AWQ:
            w = resolve(f, p + ".qweight");
            z = resolve(f, p + ".qzeros");
            s = resolve(f, p + ".scales");
            if (!w || !z || !s) return OXQ_OK;
            break;
        case OXQ_SCHEME_GPTQ:
            w = resolve(f, p + ".qweight");
            s = resolve(f, p + ".scales");
            z = resolve(f, p + ".qzeros");
            if (!w || !s) return OXQ_OK;
            break;
        case OXQ_SCHEME_COMPRESSED_TENSORS4:
            w = resolve(f, p + ".weight_packed");
            s = resolve(f, p + ".weight_scale");
            if (!w || !s) return OXQ_OK;
            break;
        default: return fail(OXQ_ERR_ARG, "oxq_safetensors_try_get_quant: bad scheme kind %d", scheme->kind);
        }
        fill(*w, qweight);
        fill(*s, scales);
        if (z) fill(*z, qzeros);
        *found = 1;
        return OXQ_OK;
    });
}

int oxq_upload(oxq_ctx *ctx, void *stream, void *dst_device, const void *src_host, uint64_t nbytes) {
    return guarded("oxq_upload", [&]() -> int {
        if (!ctx) return fail(OXQ_ERR_ARG, "oxq_upload: ctx is NULL");
        if (ctx->plan_only) return fail(OXQ_ERR_DEVICE, "oxq_upload: a plan-only ctx has no device");
        if (nbytes == 0) return OXQ_OK;
        if (!dst_device || !src_host) return fail(OXQ_ERR_ARG, "oxq_upload: NULL pointer");
        OXQ_HIP_CHECK(hipSetDevice(ctx->device));
        hipStream_t s = static_cast<hipStream_t>(stream);
        OXQ_HIP_CHECK(hipMemcpyAsync(dst_device, src_host, size_t(nbytes), hipMemcpyHostToDevice, s));
        // pageable source: the runtime stages it, but the mapping may be closed right after the call
        OXQ_HIP_CHECK(hipStreamSynchronize(s));
        return OXQ_OK;
    });
}

}  // extern "C"
