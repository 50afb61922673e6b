// GGUF container reader (host only): maps a .gguf file, parses header, metadata and tensor
// infos with bounds checks on every read, and copies tensor payloads out of the mapping with
// several threads (into pinned host memory, for example).  Takes the place of gguf.GGUFReader
// as the reference uses it (src/sensenova_u1/utils/gguf_loader.py:29-44: iterate
// reader.tensors, read name / tensor_type, copy tensor.data).
//
// File layout (GGUF v2 / v3, little endian):
//   u32 magic "GGUF" | u32 version | u64 n_tensors | u64 n_kv
//   n_kv x { string key; u32 value_type; value }          string = u64 length + bytes
//   n_tensors x { string name; u32 n_dims; u64 dims[n_dims]; u32 ggml_type; u64 offset }
//   padding to `general.alignment` (default 32) | tensor data, each at data_start + offset

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/sngguf.h"

namespace {

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF"
constexpr int64_t kDefaultAlignment = 32;
constexpr int64_t kCopyChunk = 8 << 20;

enum ValueType : uint32_t {
    VT_U8 = 0, VT_I8, VT_U16, VT_I16, VT_U32, VT_I32, VT_F32, VT_BOOL, VT_STRING, VT_ARRAY, VT_U64, VT_I64, VT_F64, VT_COUNT
};

// bytes of a scalar value type; 0 for strings / arrays / unknown
int64_t scalar_size(uint32_t t) {
    switch (t) {
    case VT_U8: case VT_I8: case VT_BOOL: return 1;
    case VT_U16: case VT_I16: return 2;
    case VT_U32: case VT_I32: case VT_F32: return 4;
    case VT_U64: case VT_I64: case VT_F64: return 8;
    default: return 0;
    }
}

// ggml type -> (elements per block, bytes per block) for the types whose size is fixed by the
// format definition; 0 for unknown ones
bool type_traits(int32_t t, int64_t& block, int64_t& bytes) {
    switch (t) {
    case 0: block = 1; bytes = 4; return true;      // F32
    case 1: block = 1; bytes = 2; return true;      // F16
    case 2: block = 32; bytes = 18; return true;    // Q4_0
    case 3: block = 32; bytes = 20; return true;    // Q4_1
    case 6: block = 32; bytes = 22; return true;    // Q5_0
    case 7: block = 32; bytes = 24; return true;    // Q5_1
    case 8: block = 32; bytes = 34; return true;    // Q8_0
    case 9: block = 32; bytes = 36; return true;    // Q8_1
    case 10: block = 256; bytes = 84; return true;  // Q2_K
    case 11: block = 256; bytes = 110; return true; // Q3_K
    case 12: block = 256; bytes = 144; return true; // Q4_K
    case 13: block = 256; bytes = 176; return true; // Q5_K
    case 14: block = 256; bytes = 210; return true; // Q6_K
    case 15: block = 256; bytes = 292; return true; // Q8_K
    case 24: block = 1; bytes = 1; return true;     // I8
    case 25: block = 1; bytes = 2; return true;     // I16
    case 26: block = 1; bytes = 4; return true;     // I32
    case 27: block = 1; bytes = 8; return true;     // I64
    case 28: block = 1; bytes = 8; return true;     // F64
    case 30: block = 1; bytes = 2; return true;     // BF16
    default: return false;
    }
}

struct Tensor {
    std::string name;
    int32_t ggml_type = 0;
    int32_t n_dims = 0;
    int64_t dims[4] = {1, 1, 1, 1};
    int64_t n_elements = 0, n_bytes = 0, file_offset = 0;
};

struct Metadata {
    std::string key;
    int32_t value_type = 0, item_type = -1;
    int64_t count = 1;
    int64_t value_offset = 0, value_bytes = 0;
};

}  // namespace

struct sngguf_file {
    int fd = -1;
    const uint8_t* map = nullptr;
    int64_t size = 0;
    int version = 0;
    int64_t alignment = kDefaultAlignment;
    int64_t data_start = 0;
    std::vector<Tensor> tensors;
    std::vector<Metadata> metadata;
};

namespace {

struct ParseError {
    int code;
    std::string message;
};

[[noreturn]] void fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    throw ParseError{code, buf};
}

// Bounds-checked little-endian cursor over the mapping.
struct Cursor {
    const uint8_t* base;
    int64_t size, pos;

    void need(int64_t n) const {
        if (n < 0 || n > size - pos) fail(SNGGUF_E_FORMAT, "truncated or corrupt GGUF file (read of %lld bytes at offset %lld, file has %lld)",
                                          (long long)n, (long long)pos, (long long)size);
    }
    template <typename T> T get() {
        need((int64_t)sizeof(T));
        T v;
        memcpy(&v, base + pos, sizeof(T));
        pos += (int64_t)sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (n > (uint64_t)(size - pos)) fail(SNGGUF_E_FORMAT, "truncated or corrupt GGUF file (string of %llu bytes at offset %lld)",
                                            (unsigned long long)n, (long long)pos);
        std::string s(reinterpret_cast<const char*>(base + pos), (size_t)n);
        pos += (int64_t)n;
        return s;
    }
    // skips one value of type t; nesting depth bounded
    void skip_value(uint32_t t, int depth) {
        if (t == VT_STRING) {
            const uint64_t n = get<uint64_t>();
            if (n > (uint64_t)(size - pos)) fail(SNGGUF_E_FORMAT, "truncated or corrupt GGUF file (string value at offset %lld)", (long long)pos);
            pos += (int64_t)n;
        } else if (t == VT_ARRAY) {
            if (depth > 4) fail(SNGGUF_E_FORMAT, "corrupt GGUF file (arrays nested too deeply)");
            const uint32_t item = get<uint32_t>();
            const uint64_t count = get<uint64_t>();
            const int64_t ss = scalar_size(item);
            if (ss) {
                if (count > (uint64_t)(size - pos) / (uint64_t)ss) fail(SNGGUF_E_FORMAT, "truncated or corrupt GGUF file (array at offset %lld)", (long long)pos);
                pos += (int64_t)count * ss;
            } else {
                if (item >= VT_COUNT) fail(SNGGUF_E_FORMAT, "corrupt GGUF file (array item type %u)", item);
                if (count > (uint64_t)(size - pos)) fail(SNGGUF_E_FORMAT, "truncated or corrupt GGUF file (array at offset %lld)", (long long)pos);
                for (uint64_t i = 0; i < count; i++) skip_value(item, depth + 1);
            }
        } else {
            const int64_t ss = scalar_size(t);
            if (!ss) fail(SNGGUF_E_FORMAT, "corrupt GGUF file (metadata value type %u)", t);
            need(ss);
            pos += ss;
        }
    }
};

void parse(sngguf_file& f, const char* path) {
    Cursor c{f.map, f.size, 0};
    if (f.size < 4 || c.get<uint32_t>() != kMagic) fail(SNGGUF_E_FORMAT, "%s: bad magic, not a GGUF file", path);
    f.version = (int)c.get<uint32_t>();
    if (f.version != 2 && f.version != 3) fail(SNGGUF_E_FORMAT, "%s: unsupported GGUF version %d", path, f.version);
    const uint64_t n_tensors = c.get<uint64_t>();
    const uint64_t n_kv = c.get<uint64_t>();
    // every entry takes at least 12 (kv) / 24 (tensor) bytes: bounds the reserve below
    if (n_kv > (uint64_t)f.size / 12 || n_tensors > (uint64_t)f.size / 24) fail(SNGGUF_E_FORMAT, "%s: truncated or corrupt GGUF file (entry counts)", path);
    f.metadata.reserve((size_t)n_kv);
    for (uint64_t i = 0; i < n_kv; i++) {
        Metadata m;
        m.key = c.str();
        m.value_type = (int32_t)c.get<uint32_t>();
        m.value_offset = c.pos;
        if ((uint32_t)m.value_type == VT_ARRAY) {
            Cursor peek = c;
            m.item_type = (int32_t)peek.get<uint32_t>();
            m.count = (int64_t)peek.get<uint64_t>();
        } else if ((uint32_t)m.value_type == VT_STRING) {
            Cursor peek = c;
            m.count = (int64_t)peek.get<uint64_t>();
        }
        c.skip_value((uint32_t)m.value_type, 0);
        m.value_bytes = c.pos - m.value_offset;
        if (m.key == "general.alignment") {
            const int64_t ss = scalar_size((uint32_t)m.value_type);
            if (ss == 0 || ss > 8) fail(SNGGUF_E_FORMAT, "%s: general.alignment is not an integer", path);
            uint64_t v = 0;
            memcpy(&v, f.map + m.value_offset, (size_t)ss);
            if (v == 0 || v > (1u << 20) || (v & (v - 1)) != 0) fail(SNGGUF_E_FORMAT, "%s: general.alignment %llu is not a power of two", path, (unsigned long long)v);
            f.alignment = (int64_t)v;
        }
        f.metadata.push_back(std::move(m));
    }
    struct Raw { uint64_t offset; };
    std::vector<Raw> raw;
    raw.reserve((size_t)n_tensors);
    f.tensors.reserve((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; i++) {
        Tensor t;
        t.name = c.str();
        const uint32_t nd = c.get<uint32_t>();
        if (nd > 4) fail(SNGGUF_E_FORMAT, "%s: tensor %s has %u dimensions", path, t.name.c_str(), nd);
        t.n_dims = (int32_t)nd;
        for (uint32_t d = 0; d < nd; d++) {
            const uint64_t v = c.get<uint64_t>();
            if (v > (uint64_t)INT64_MAX) fail(SNGGUF_E_FORMAT, "%s: tensor %s: dimension too large", path, t.name.c_str());
            t.dims[d] = (int64_t)v;
        }
        t.ggml_type = (int32_t)c.get<uint32_t>();
        raw.push_back({c.get<uint64_t>()});
        f.tensors.push_back(std::move(t));
    }
    f.data_start = (c.pos + f.alignment - 1) / f.alignment * f.alignment;
    for (size_t i = 0; i < f.tensors.size(); i++) {
        Tensor& t = f.tensors[i];
        int64_t block, bytes;
        if (!type_traits(t.ggml_type, block, bytes))
            fail(SNGGUF_E_FORMAT, "%s: tensor %s has ggml type %d whose block size is not known", path, t.name.c_str(), t.ggml_type);
        unsigned __int128 n = 1;
        for (int d = 0; d < t.n_dims; d++) {
            n *= (unsigned __int128)t.dims[d];
            if (n > (unsigned __int128)INT64_MAX) fail(SNGGUF_E_FORMAT, "%s: tensor %s: element count overflows", path, t.name.c_str());
        }
        t.n_elements = (int64_t)n;
        if (t.n_dims > 0 && t.dims[0] % block != 0)
            fail(SNGGUF_E_FORMAT, "%s: tensor %s: row length %lld is not a multiple of block size %lld", path, t.name.c_str(),
                 (long long)t.dims[0], (long long)block);
        const unsigned __int128 nb = (unsigned __int128)(t.n_elements / block) * (unsigned __int128)bytes;
        const unsigned __int128 start = (unsigned __int128)f.data_start + raw[i].offset;
        if (start + nb > (unsigned __int128)f.size) fail(SNGGUF_E_FORMAT, "%s: tensor %s runs past the end of the file", path, t.name.c_str());
        t.n_bytes = (int64_t)nb;
        t.file_offset = (int64_t)start;
    }
}

void set_error(char* err, int64_t err_len, const std::string& msg) {
    if (!err || err_len <= 0) return;
    const size_t n = msg.size() < (size_t)err_len - 1 ? msg.size() : (size_t)err_len - 1;
    memcpy(err, msg.data(), n);
    err[n] = 0;
}

}  // namespace

extern "C" {

int sngguf_file_open(const char* path, sngguf_file** out, char* err, int64_t err_len) {
    if (out) *out = nullptr;
    if (!path || !out) {
        set_error(err, err_len, "path or out is NULL");
        return SNGGUF_E_NULLPTR;
    }
    sngguf_file* f = new sngguf_file();
    int code = SNGGUF_OK;
    std::string msg;
    f->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (f->fd < 0 || fstat(f->fd, &st) != 0) {
        code = SNGGUF_E_IO;
        msg = std::string(path) + ": cannot open: " + strerror(errno);
    } else if (st.st_size == 0) {
        code = SNGGUF_E_FORMAT;
        msg = std::string(path) + ": not a GGUF file (empty)";
    } else {
        f->size = (int64_t)st.st_size;
        void* p = mmap(nullptr, (size_t)f->size, PROT_READ, MAP_PRIVATE, f->fd, 0);
        if (p == MAP_FAILED) {
            code = SNGGUF_E_IO;
            msg = std::string(path) + ": cannot map: " + strerror(errno);
        } else {
            f->map = static_cast<const uint8_t*>(p);
            try {
                parse(*f, path);
            } catch (const ParseError& e) {
                code = e.code;
                msg = e.message;
            } catch (const std::exception& e) {
                code = SNGGUF_E_FORMAT;
                msg = std::string(path) + ": " + e.what();
            }
        }
    }
    if (code != SNGGUF_OK) {
        set_error(err, err_len, msg);
        sngguf_file_close(f);
        return code;
    }
    *out = f;
    return SNGGUF_OK;
}

void sngguf_file_close(sngguf_file* f) {
    if (!f) return;
    if (f->map) munmap(const_cast<uint8_t*>(f->map), (size_t)f->size);
    if (f->fd >= 0) close(f->fd);
    delete f;
}

int sngguf_file_version(const sngguf_file* f) { return f ? f->version : 0; }
int64_t sngguf_file_alignment(const sngguf_file* f) { return f ? f->alignment : 0; }
int64_t sngguf_file_tensor_count(const sngguf_file* f) { return f ? (int64_t)f->tensors.size() : 0; }
int64_t sngguf_file_metadata_count(const sngguf_file* f) { return f ? (int64_t)f->metadata.size() : 0; }

int sngguf_file_tensor(const sngguf_file* f, int64_t index, sngguf_tensor_info* out) {
    if (!f || !out) return SNGGUF_E_NULLPTR;
    if (index < 0 || index >= (int64_t)f->tensors.size()) return SNGGUF_E_BADSHAPE;
    const Tensor& t = f->tensors[(size_t)index];
    out->name = t.name.c_str();
    out->ggml_type = t.ggml_type;
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) out->dims[d] = t.dims[d];
    out->n_elements = t.n_elements;
    out->n_bytes = t.n_bytes;
    out->file_offset = t.file_offset;
    out->data = f->map + t.file_offset;
    return SNGGUF_OK;
}

int sngguf_file_metadata(const sngguf_file* f, int64_t index, sngguf_metadata_info* out) {
    if (!f || !out) return SNGGUF_E_NULLPTR;
    if (index < 0 || index >= (int64_t)f->metadata.size()) return SNGGUF_E_BADSHAPE;
    const Metadata& m = f->metadata[(size_t)index];
    out->key = m.key.c_str();
    out->value_type = m.value_type;
    out->item_type = m.item_type;
    out->count = m.count;
    out->value = f->map + m.value_offset;
    out->value_bytes = m.value_bytes;
    return SNGGUF_OK;
}

int sngguf_file_read_tensors(const sngguf_file* f, const int64_t* indices, void* const* dst, int64_t count, int threads) {
    if (!f || (count > 0 && (!indices || !dst))) return SNGGUF_E_NULLPTR;
    if (count < 0) return SNGGUF_E_BADSHAPE;
    struct Piece { const uint8_t* src; uint8_t* dst; int64_t n; };
    std::vector<Piece> pieces;
    for (int64_t i = 0; i < count; i++) {
        if (indices[i] < 0 || indices[i] >= (int64_t)f->tensors.size()) return SNGGUF_E_BADSHAPE;
        const Tensor& t = f->tensors[(size_t)indices[i]];
        if (t.n_bytes > 0 && !dst[i]) return SNGGUF_E_NULLPTR;
        for (int64_t o = 0; o < t.n_bytes; o += kCopyChunk) {
            const int64_t n = t.n_bytes - o < kCopyChunk ? t.n_bytes - o : kCopyChunk;
            pieces.push_back({f->map + t.file_offset + o, static_cast<uint8_t*>(dst[i]) + o, n});
        }
    }
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    if ((int64_t)threads > (int64_t)pieces.size()) threads = (int)pieces.size();
    std::atomic<size_t> next{0};
    auto work = [&]() {
        for (size_t i = next.fetch_add(1); i < pieces.size(); i = next.fetch_add(1)) memcpy(pieces[i].dst, pieces[i].src, (size_t)pieces[i].n);
    };
    if (threads <= 1) {
        work();
        return SNGGUF_OK;
    }
    std::vector<std::thread> pool;
    try {
        for (int t = 1; t < threads; t++) pool.emplace_back(work);
    } catch (...) {
        // could not start every helper: the ones that did start and this thread finish the job
    }
    work();
    for (auto& th : pool) th.join();
    return SNGGUF_OK;
}

}  // extern "C"
