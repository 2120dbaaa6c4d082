// GGUF v3 reader and DFlash drafter loader (host only; no device code in this file).
//
// Follows GgufFile (crates/qwen-llm/src/gguf.rs:129-740, layout and validation :790-940, :1303-1600,
// split files :154-228 and :954-1095) and open_dflash_drafter_for_target
// (crates/qwen-llm/src/loader.rs:832-1290).  Each file is mapped read-only; every read of a header is
// bounds-checked against its mapping; tensor bytes are never copied (callers upload straight from the
// mapping).  A split model is one handle: the first shard's metadata, the tensors of every shard.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/dflash_hip.h"

namespace {

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF", little-endian
constexpr uint64_t kDefaultAlignment = 32, kMaxAlignment = 65536;
constexpr uint64_t kMaxTensors = 1000000, kMaxKv = 1000000, kMaxKeyLen = 1024, kMaxTensorNameLen = 64;
constexpr uint64_t kMaxStringLen = 100ull << 20, kMaxArrayLen = 10000000, kMaxDimension = 1ull << 30;
constexpr uint64_t kMaxElements = 1ull << 40;
constexpr uint64_t kMaxSplits = 1024;  // gguf.rs:42
// loader caps (loader.rs:104-107)
constexpr uint32_t kMaxArchLayers = 4096, kMaxArchDim = 1u << 20, kMaxBlockSize = 4096;
constexpr uint64_t kMaxKernelDim = 1ull << 20;

// GGUF metadata value types
enum : uint32_t { T_U8 = 0, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 };

struct Value {
    uint32_t type = 0;       // scalar type, or T_ARR
    uint32_t item_type = 0;  // arrays
    uint64_t len = 0;        // arrays: elements; strings: bytes
    size_t at = 0;           // file offset of the payload (string bytes / first array item / scalar)
};

struct Tensor {
    std::string name;
    dflash_gguf_tensor d;
};

// elements per block and bytes per block of a ggml type; false for an id this reader does not know
bool type_block(uint32_t t, uint64_t *elems, uint64_t *bytes) {
    struct Row {
        uint32_t id;
        uint32_t elems, bytes;
    };
    static const Row rows[] = {
        {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},    {7, 32, 24},    {8, 32, 34},
        {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292},
        {16, 256, 66},  {17, 256, 74},  {18, 256, 98},  {19, 256, 50},  {20, 32, 18},   {21, 256, 110}, {22, 256, 82},
        {23, 256, 136}, {24, 1, 1},     {25, 1, 2},     {26, 1, 4},     {27, 1, 8},     {28, 1, 8},     {29, 256, 56},
        {30, 1, 2},     {34, 256, 54},  {35, 256, 66},  {39, 32, 17},
    };
    for (const Row &r : rows)
        if (r.id == t) {
            *elems = r.elems;
            *bytes = r.bytes;
            return true;
        }
    return false;
}

}  // namespace

struct dflash_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    size_t size = 0;
    uint64_t alignment = kDefaultAlignment, data_start = 0;
    std::unordered_map<std::string, Value> kv;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, size_t> by_name;
    std::vector<dflash_gguf *> more;  // shards 1.. of a split model (their tensors are merged into `tensors`)
    mutable std::string err;
};

namespace {

int32_t fail(const dflash_gguf *g, int32_t status, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g->err = buf;
    return status;
}

// Cursor over the mapping; every read checks the bounds first (gguf.rs:1490-1506, :1560-1568).
struct Reader {
    const dflash_gguf *g;
    size_t p = 0;
    bool ok = true;
    bool need(uint64_t n) {
        if (!ok) return false;
        if (n > g->size || p > g->size - n) {
            fail(g, DFLASH_ERR_FORMAT, "out-of-bounds read at offset %zu (len %llu, file size %zu)", p,
                 static_cast<unsigned long long>(n), g->size);
            ok = false;
        }
        return ok;
    }
    template <typename T>
    T get() {
        T v{};
        if (need(sizeof(T))) {
            memcpy(&v, g->map + p, sizeof(T));
            p += sizeof(T);
        }
        return v;
    }
    bool bad(const char *fmt, ...) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof(buf), fmt, ap);
        va_end(ap);
        g->err = buf;
        ok = false;
        return false;
    }
};

size_t scalar_size(uint32_t t) {
    switch (t) {
    case T_U8: case T_I8: case T_BOOL: return 1;
    case T_U16: case T_I16: return 2;
    case T_U32: case T_I32: case T_F32: return 4;
    case T_U64: case T_I64: case T_F64: return 8;
    default: return 0;
    }
}

// Reads (and skips) one value of `type` (skip_value, gguf.rs:1508-1558).
bool read_value(Reader &r, uint32_t type, Value *out) {
    out->type = type;
    if (const size_t n = scalar_size(type)) {
        out->at = r.p;
        if (!r.need(n)) return false;
        r.p += n;
        return true;
    }
    if (type == T_STR) {
        const uint64_t len = r.get<uint64_t>();
        if (!r.ok) return false;
        if (len > kMaxStringLen) return r.bad("absurd string length %llu at offset %zu", static_cast<unsigned long long>(len), r.p);
        out->at = r.p;
        out->len = len;
        if (!r.need(len)) return false;
        r.p += len;
        return true;
    }
    if (type == T_ARR) {
        const uint32_t item = r.get<uint32_t>();
        const uint64_t len = r.get<uint64_t>();
        if (!r.ok) return false;
        if (item == T_ARR) return r.bad("nested metadata arrays are not supported");
        if (item > T_F64) return r.bad("unknown metadata value type %u", item);
        if (len > kMaxArrayLen) return r.bad("absurd array length %llu at offset %zu", static_cast<unsigned long long>(len), r.p);
        out->item_type = item;
        out->len = len;
        out->at = r.p;
        if (const size_t n = scalar_size(item)) {
            if (!r.need(len * n)) return false;
            r.p += len * n;
            return true;
        }
        for (uint64_t i = 0; i < len; i++) {  // strings
            Value tmp;
            if (!read_value(r, T_STR, &tmp)) return false;
        }
        return true;
    }
    return r.bad("unknown metadata value type %u", type);
}

bool valid_utf8(const uint8_t *s, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = s[i];
        size_t extra = 0;
        uint32_t cp = 0;
        if (c < 0x80) { i++; continue; }
        else if ((c & 0xE0) == 0xC0) { extra = 1; cp = c & 0x1F; }
        else if ((c & 0xF0) == 0xE0) { extra = 2; cp = c & 0x0F; }
        else if ((c & 0xF8) == 0xF0) { extra = 3; cp = c & 0x07; }
        else return false;
        if (i + extra >= n) return false;
        for (size_t k = 1; k <= extra; k++) {
            if ((s[i + k] & 0xC0) != 0x80) return false;
            cp = (cp << 6) | (s[i + k] & 0x3F);
        }
        if ((extra == 1 && cp < 0x80) || (extra == 2 && cp < 0x800) || (extra == 3 && (cp < 0x10000 || cp > 0x10FFFF)) ||
            (cp >= 0xD800 && cp <= 0xDFFF))
            return false;
        i += extra + 1;
    }
    return true;
}

// scalar at `at` of integer type `t` as a non-negative u64
bool int_as_u64(const dflash_gguf *g, uint32_t t, size_t at, uint64_t *out) {
    const uint8_t *p = g->map + at;
    int64_t sv = 0;
    switch (t) {
    case T_U8: *out = *p; return true;
    case T_U16: { uint16_t v; memcpy(&v, p, 2); *out = v; return true; }
    case T_U32: { uint32_t v; memcpy(&v, p, 4); *out = v; return true; }
    case T_U64: { uint64_t v; memcpy(&v, p, 8); *out = v; return true; }
    case T_I8: sv = static_cast<int8_t>(*p); break;
    case T_I16: { int16_t v; memcpy(&v, p, 2); sv = v; break; }
    case T_I32: { int32_t v; memcpy(&v, p, 4); sv = v; break; }
    case T_I64: { int64_t v; memcpy(&v, p, 8); sv = v; break; }
    default: return false;
    }
    if (sv < 0) return false;
    *out = static_cast<uint64_t>(sv);
    return true;
}

bool float_as_f64(const dflash_gguf *g, uint32_t t, size_t at, double *out) {
    if (t == T_F32) { float v; memcpy(&v, g->map + at, 4); *out = v; return true; }
    if (t == T_F64) { memcpy(out, g->map + at, 8); return true; }
    return false;
}

int32_t parse(dflash_gguf *g) {
    Reader r{g};
    const uint32_t magic = r.get<uint32_t>();
    if (!r.ok) return DFLASH_ERR_FORMAT;
    if (magic != kMagic) return fail(g, DFLASH_ERR_FORMAT, "bad magic: not a GGUF file");
    const uint32_t version = r.get<uint32_t>();
    if (!r.ok) return DFLASH_ERR_FORMAT;
    if (version != 3) return fail(g, DFLASH_ERR_FORMAT, "unsupported GGUF version %u (only v3 supported)", version);
    const uint64_t n_tensors = r.get<uint64_t>(), n_kv = r.get<uint64_t>();
    if (!r.ok) return DFLASH_ERR_FORMAT;
    if (n_tensors > kMaxTensors) return fail(g, DFLASH_ERR_FORMAT, "absurd tensor count: %llu", static_cast<unsigned long long>(n_tensors));
    if (n_kv > kMaxKv) return fail(g, DFLASH_ERR_FORMAT, "absurd kv count: %llu", static_cast<unsigned long long>(n_kv));

    for (uint64_t i = 0; i < n_kv; i++) {
        const uint64_t klen = r.get<uint64_t>();
        if (!r.ok) return DFLASH_ERR_FORMAT;
        if (klen == 0) return fail(g, DFLASH_ERR_FORMAT, "metadata key has zero length");
        if (klen > kMaxKeyLen) return fail(g, DFLASH_ERR_FORMAT, "metadata key length %llu exceeds %llu", static_cast<unsigned long long>(klen), static_cast<unsigned long long>(kMaxKeyLen));
        if (!r.need(klen)) return DFLASH_ERR_FORMAT;
        if (!valid_utf8(g->map + r.p, klen)) return fail(g, DFLASH_ERR_FORMAT, "metadata key not valid UTF-8");
        std::string key(reinterpret_cast<const char *>(g->map + r.p), klen);
        r.p += klen;
        const uint32_t type = r.get<uint32_t>();
        Value v;
        if (!r.ok || !read_value(r, type, &v)) return DFLASH_ERR_FORMAT;
        if (!g->kv.emplace(key, v).second) return fail(g, DFLASH_ERR_FORMAT, "duplicate metadata key \"%s\"", key.c_str());
    }

    // general.alignment (gguf.rs:810-838): must be an integer in 1..=65536 when present
    auto al = g->kv.find("general.alignment");
    if (al != g->kv.end()) {
        uint64_t a = 0;
        if (!int_as_u64(g, al->second.type, al->second.at, &a) || a == 0 || a > kMaxAlignment)
            return fail(g, DFLASH_ERR_FORMAT, "general.alignment out of range (1..=%llu)", static_cast<unsigned long long>(kMaxAlignment));
        g->alignment = a;
    }

    struct Raw {
        uint64_t offset;
    };
    std::vector<Raw> raw;
    g->tensors.reserve(std::min<uint64_t>(n_tensors, g->size / 33));  // a table entry is at least 33 bytes
    for (uint64_t i = 0; i < n_tensors; i++) {
        const uint64_t nlen = r.get<uint64_t>();
        if (!r.ok) return DFLASH_ERR_FORMAT;
        if (nlen == 0) return fail(g, DFLASH_ERR_FORMAT, "tensor name has zero length");
        if (nlen > kMaxTensorNameLen) return fail(g, DFLASH_ERR_FORMAT, "tensor name length %llu exceeds %llu", static_cast<unsigned long long>(nlen), static_cast<unsigned long long>(kMaxTensorNameLen));
        if (!r.need(nlen)) return DFLASH_ERR_FORMAT;
        if (!valid_utf8(g->map + r.p, nlen)) return fail(g, DFLASH_ERR_FORMAT, "tensor name not valid UTF-8");
        Tensor t;
        t.name.assign(reinterpret_cast<const char *>(g->map + r.p), nlen);
        r.p += nlen;
        const uint32_t n_dims = r.get<uint32_t>();
        if (!r.ok) return DFLASH_ERR_FORMAT;
        if (n_dims == 0 || n_dims > 4)
            return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" declares %u dimensions (must be 1..=4)", t.name.c_str(), n_dims);
        memset(&t.d, 0, sizeof(t.d));
        uint64_t shape[4] = {1, 1, 1, 1};
        for (uint32_t d = 0; d < n_dims; d++) shape[d] = r.get<uint64_t>();
        const uint32_t type = r.get<uint32_t>();
        const uint64_t offset = r.get<uint64_t>();
        if (!r.ok) return DFLASH_ERR_FORMAT;
        uint32_t rank = n_dims;
        while (rank > 1 && shape[rank - 1] == 1) rank--;  // trailing 1s are not dimensions
        uint64_t elements = 1;
        for (uint32_t d = 0; d < rank; d++) {
            if (shape[d] == 0) return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" has a zero-length dimension", t.name.c_str());
            if (shape[d] > kMaxDimension)
                return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" dimension %llu exceeds %llu", t.name.c_str(), static_cast<unsigned long long>(shape[d]), static_cast<unsigned long long>(kMaxDimension));
            if (__builtin_mul_overflow(elements, shape[d], &elements) || elements > kMaxElements)
                return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" has too many elements", t.name.c_str());
        }
        uint64_t be = 0, bb = 0;
        if (!type_block(type, &be, &bb)) return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" has unknown type %u", t.name.c_str(), type);
        if (shape[0] % be) return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\": row length %llu is not a multiple of the block size %llu", t.name.c_str(), static_cast<unsigned long long>(shape[0]), static_cast<unsigned long long>(be));
        t.d.type = static_cast<int32_t>(type);
        t.d.n_dims = static_cast<int32_t>(rank);
        for (uint32_t d = 0; d < 4; d++) t.d.shape[d] = d < rank ? shape[d] : 1;
        t.d.n_bytes = elements / be * bb;
        if (!g->by_name.emplace(t.name, g->tensors.size()).second)
            return fail(g, DFLASH_ERR_FORMAT, "duplicate tensor name \"%s\"", t.name.c_str());
        g->tensors.push_back(t);
        raw.push_back({offset});
    }

    // tensor data starts at the next multiple of the alignment (gguf.rs:1460-1480)
    const uint64_t end = r.p;
    const uint64_t aligned = (end + g->alignment - 1) / g->alignment * g->alignment;
    if (aligned > g->size) {
        if (g->tensors.empty() && end == g->size) {
            g->data_start = end;
            return DFLASH_OK;
        }
        return fail(g, DFLASH_ERR_FORMAT, "aligned header end %llu > file size %zu", static_cast<unsigned long long>(aligned), g->size);
    }
    g->data_start = aligned;
    for (size_t i = 0; i < g->tensors.size(); i++) {
        Tensor &t = g->tensors[i];
        if (raw[i].offset % g->alignment)
            return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" offset %llu not aligned to %llu", t.name.c_str(), static_cast<unsigned long long>(raw[i].offset), static_cast<unsigned long long>(g->alignment));
        if (raw[i].offset > g->size - aligned || t.d.n_bytes > g->size - aligned - raw[i].offset)
            return fail(g, DFLASH_ERR_FORMAT, "tensor \"%s\" (offset %llu, size %llu) runs past the end of the file", t.name.c_str(), static_cast<unsigned long long>(raw[i].offset), static_cast<unsigned long long>(t.d.n_bytes));
        t.d.data_host = g->map + aligned + raw[i].offset;
    }
    // no two tensors overlap (gguf.rs:916-932)
    std::vector<size_t> order(g->tensors.size());
    for (size_t i = 0; i < order.size(); i++) order[i] = i;
    std::sort(order.begin(), order.end(), [&](size_t a, size_t b) { return raw[a].offset < raw[b].offset; });
    for (size_t i = 1; i < order.size(); i++) {
        const Tensor &a = g->tensors[order[i - 1]], &b = g->tensors[order[i]];
        if (raw[order[i - 1]].offset + a.d.n_bytes > raw[order[i]].offset)
            return fail(g, DFLASH_ERR_FORMAT, "tensors \"%s\" and \"%s\" have overlapping data ranges", a.name.c_str(), b.name.c_str());
    }
    return DFLASH_OK;
}

const Value *find_kv(const dflash_gguf *g, const char *key) {
    if (!g || !key) return nullptr;
    auto it = g->kv.find(key);
    return it == g->kv.end() ? nullptr : &it->second;
}

}  // namespace

namespace {

// Maps and parses one file.  On failure the message is in *msg and nothing stays open.
int32_t open_one(const char *path, dflash_gguf **out, std::string *msg) {
    dflash_gguf *g = new dflash_gguf();
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (g->fd < 0 || fstat(g->fd, &st) != 0 || !S_ISREG(st.st_mode)) {
        *msg = std::string("cannot open ") + path + ": " + (g->fd < 0 ? strerror(errno) : "not a regular file");
        dflash_gguf_close(g);
        return DFLASH_ERR_IO;
    }
    g->size = static_cast<size_t>(st.st_size);
    if (g->size) {
        void *m = mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
        if (m == MAP_FAILED) {
            *msg = std::string("mmap failed: ") + strerror(errno);
            g->map = nullptr;
            dflash_gguf_close(g);
            return DFLASH_ERR_IO;
        }
        g->map = static_cast<const uint8_t *>(m);
    }
    int32_t rc;
    try {
        rc = parse(g);
    } catch (const std::exception &e) {  // allocation failure while building the tables
        rc = fail(g, DFLASH_ERR_IO, "out of memory while reading the header (%s)", e.what());
    }
    if (rc) {
        *msg = g->err;
        dflash_gguf_close(g);
        return rc;
    }
    *out = g;
    return DFLASH_OK;
}

bool kv_u64(const dflash_gguf *g, const char *key, uint64_t *out) {
    const Value *v = find_kv(g, key);
    return v && int_as_u64(g, v->type, v->at, out);
}

std::string split_suffix(uint64_t no, uint64_t count) {  // gguf.rs:985: shard numbers in names are 1-based
    char buf[64];
    snprintf(buf, sizeof(buf), "-%05llu-of-%05llu.gguf", static_cast<unsigned long long>(no + 1), static_cast<unsigned long long>(count));
    return buf;
}

std::string fmt(const char *f, ...) {
    char buf[768];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof(buf), f, ap);
    va_end(ap);
    return buf;
}

// The rest of a split model, `first` being its shard 0 (GgufFile::open, gguf.rs:154-228): the siblings are named
// by the first file's own suffix; each must carry its own number, the same count and (when present) the same
// total; tensors are appended shard by shard, never past the declared total, and a name may appear once.
int32_t open_split(dflash_gguf *first, const char *path, uint64_t count, std::string *msg) {
    using ull = unsigned long long;
    if (count > kMaxSplits) return *msg = fmt("split.count %llu in %s exceeds cap %llu", (ull)count, path, (ull)kMaxSplits), DFLASH_ERR_FORMAT;
    uint64_t no = 0, total = 0;
    if (!kv_u64(first, "split.no", &no)) return *msg = fmt("missing \"split.no\" in split GGUF %s", path), DFLASH_ERR_FORMAT;
    if (no != 0)
        return *msg = fmt("illegal split file idx %llu (file: %s), model must be loaded with the first split", (ull)no, path), DFLASH_ERR_FORMAT;
    if (!kv_u64(first, "split.tensors.count", &total))
        return *msg = fmt("missing \"split.tensors.count\" in split GGUF %s", path), DFLASH_ERR_FORMAT;
    if (total > kMaxTensors) return *msg = fmt("split.tensors.count %llu in %s exceeds cap %llu", (ull)total, path, (ull)kMaxTensors), DFLASH_ERR_FORMAT;
    const std::string p(path), suffix = split_suffix(0, count);
    if (p.size() < suffix.size() || p.compare(p.size() - suffix.size(), suffix.size(), suffix) != 0)
        return *msg = fmt("invalid split file name: %s (expected suffix \"%s\")", path, suffix.c_str()), DFLASH_ERR_FORMAT;
    const std::string prefix = p.substr(0, p.size() - suffix.size());
    if (prefix.empty()) return *msg = fmt("invalid split file: %s", path), DFLASH_ERR_FORMAT;
    if (first->tensors.size() > total)
        return *msg = fmt("split shards declare %llu tensors but at least %zu were found", (ull)total, first->tensors.size()), DFLASH_ERR_FORMAT;
    for (uint64_t idx = 1; idx < count; idx++) {
        const std::string sp = prefix + split_suffix(idx, count);
        dflash_gguf *s = nullptr;
        if (const int32_t rc = open_one(sp.c_str(), &s, msg)) return rc;
        first->more.push_back(s);  // owned from here on: closed with `first`
        uint64_t got = 0;
        if (!kv_u64(s, "split.no", &got)) return *msg = fmt("missing \"split.no\" in GGUF split %s", sp.c_str()), DFLASH_ERR_FORMAT;
        if (got != idx) return *msg = fmt("invalid split file idx: %llu (file: %s), expected %llu", (ull)got, sp.c_str(), (ull)idx), DFLASH_ERR_FORMAT;
        if (!kv_u64(s, "split.count", &got)) return *msg = fmt("missing \"split.count\" in GGUF split %s", sp.c_str()), DFLASH_ERR_FORMAT;
        if (got > kMaxSplits) return *msg = fmt("split.count %llu in %s exceeds cap %llu", (ull)got, sp.c_str(), (ull)kMaxSplits), DFLASH_ERR_FORMAT;
        if (got != count) return *msg = fmt("invalid split count: %llu (file: %s), expected %llu", (ull)got, sp.c_str(), (ull)count), DFLASH_ERR_FORMAT;
        if (find_kv(s, "split.tensors.count") && kv_u64(s, "split.tensors.count", &got)) {
            if (got > kMaxTensors) return *msg = fmt("split.tensors.count %llu in %s exceeds cap %llu", (ull)got, sp.c_str(), (ull)kMaxTensors), DFLASH_ERR_FORMAT;
            if (got != total) return *msg = fmt("invalid split tensor count: %llu (file: %s), expected %llu", (ull)got, sp.c_str(), (ull)total), DFLASH_ERR_FORMAT;
        }
        if (first->tensors.size() + s->tensors.size() > total)
            return *msg = fmt("split shards declare %llu tensors but at least %zu were found", (ull)total, first->tensors.size() + s->tensors.size()), DFLASH_ERR_FORMAT;
        for (const Tensor &t : s->tensors) {
            if (!first->by_name.emplace(t.name, first->tensors.size()).second)
                return *msg = fmt("invalid model: tensor \"%s\" is duplicated across GGUF splits", t.name.c_str()), DFLASH_ERR_FORMAT;
            first->tensors.push_back(t);  // data_host points into the sibling's mapping, which lives as long as `first`
        }
    }
    if (first->tensors.size() != total)
        return *msg = fmt("corrupted split model: %llu tensors expected but %zu found", (ull)total, first->tensors.size()), DFLASH_ERR_FORMAT;
    return DFLASH_OK;
}

}  // namespace

extern "C" int32_t dflash_gguf_open(const char *path, dflash_gguf **out, char *err, size_t err_cap) {
    auto say = [&](const std::string &m) {
        if (err && err_cap) snprintf(err, err_cap, "%s", m.c_str());
    };
    if (out) *out = nullptr;
    if (!path || !out) {
        say("null argument");
        return DFLASH_ERR_INVALID_INPUT;
    }
    dflash_gguf *g = nullptr;
    std::string msg;
    int32_t rc;
    try {
        rc = open_one(path, &g, &msg);
        uint64_t count = 0;
        if (!rc && kv_u64(g, "split.count", &count) && count > 1) rc = open_split(g, path, count, &msg);
    } catch (const std::exception &e) {  // allocation failure: nothing may cross the C boundary
        rc = DFLASH_ERR_IO;
        msg = std::string("out of memory while reading the header (") + e.what() + ")";
    }
    if (rc) {
        say(msg);
        dflash_gguf_close(g);
        return rc;
    }
    *out = g;
    return DFLASH_OK;
}

extern "C" void dflash_gguf_close(dflash_gguf *g) {
    if (!g) return;
    for (dflash_gguf *s : g->more) dflash_gguf_close(s);
    if (g->map) munmap(const_cast<uint8_t *>(g->map), g->size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

extern "C" int64_t dflash_gguf_shard_count(const dflash_gguf *g) { return g ? static_cast<int64_t>(1 + g->more.size()) : 0; }
extern "C" const char *dflash_gguf_last_error(const dflash_gguf *g) { return g ? g->err.c_str() : "null handle"; }
extern "C" int64_t dflash_gguf_tensor_count(const dflash_gguf *g) { return g ? static_cast<int64_t>(g->tensors.size()) : 0; }
extern "C" int64_t dflash_gguf_kv_count(const dflash_gguf *g) { return g ? static_cast<int64_t>(g->kv.size()) : 0; }
extern "C" uint64_t dflash_gguf_alignment(const dflash_gguf *g) { return g ? g->alignment : 0; }
extern "C" uint64_t dflash_gguf_data_start(const dflash_gguf *g) { return g ? g->data_start : 0; }

extern "C" int32_t dflash_gguf_tensor_at(const dflash_gguf *g, int64_t i, const char **name, dflash_gguf_tensor *out) {
    if (!g) return DFLASH_ERR_INVALID_INPUT;
    if (i < 0 || i >= static_cast<int64_t>(g->tensors.size())) return fail(g, DFLASH_ERR_INVALID_INPUT, "tensor index %lld out of range", static_cast<long long>(i));
    if (name) *name = g->tensors[i].name.c_str();
    if (out) *out = g->tensors[i].d;
    return DFLASH_OK;
}

extern "C" int32_t dflash_gguf_find(const dflash_gguf *g, const char *name, dflash_gguf_tensor *out) {
    if (!g || !name) return 0;
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) return 0;
    if (out) *out = g->tensors[it->second].d;
    return 1;
}

extern "C" int32_t dflash_gguf_get_u64(const dflash_gguf *g, const char *key, uint64_t *out) {
    const Value *v = find_kv(g, key);
    uint64_t x = 0;
    if (!v || !int_as_u64(g, v->type, v->at, &x)) return 0;
    if (out) *out = x;
    return 1;
}

extern "C" int32_t dflash_gguf_get_f64(const dflash_gguf *g, const char *key, double *out) {
    const Value *v = find_kv(g, key);
    double x = 0;
    if (!v || !float_as_f64(g, v->type, v->at, &x)) return 0;
    if (out) *out = x;
    return 1;
}

extern "C" int32_t dflash_gguf_get_bool(const dflash_gguf *g, const char *key, int32_t *out) {
    const Value *v = find_kv(g, key);
    if (!v || v->type != T_BOOL) return 0;
    if (out) *out = g->map[v->at] != 0;
    return 1;
}

extern "C" int32_t dflash_gguf_get_str(const dflash_gguf *g, const char *key, const char **out, uint64_t *len) {
    const Value *v = find_kv(g, key);
    if (!v || v->type != T_STR) return 0;
    if (out) *out = reinterpret_cast<const char *>(g->map + v->at);
    if (len) *len = v->len;
    return 1;
}

extern "C" int64_t dflash_gguf_get_u64_array(const dflash_gguf *g, const char *key, uint64_t *out, int64_t cap) {
    const Value *v = find_kv(g, key);
    if (!v) return -1;
    const size_t sz = v->type == T_ARR ? scalar_size(v->item_type) : 0;
    if (!sz || v->item_type == T_F32 || v->item_type == T_F64 || v->item_type == T_BOOL) return -2;
    for (uint64_t i = 0; i < v->len; i++) {
        uint64_t x = 0;
        if (!int_as_u64(g, v->item_type, v->at + i * sz, &x)) return -2;
        if (out && static_cast<int64_t>(i) < cap) out[i] = x;
    }
    return static_cast<int64_t>(v->len);
}

extern "C" int64_t dflash_gguf_get_bool_array(const dflash_gguf *g, const char *key, uint8_t *out, int64_t cap) {
    const Value *v = find_kv(g, key);
    if (!v) return -1;
    if (v->type != T_ARR || v->item_type != T_BOOL) return -2;
    for (uint64_t i = 0; i < v->len && out && static_cast<int64_t>(i) < cap; i++) out[i] = g->map[v->at + i] != 0;
    return static_cast<int64_t>(v->len);
}

extern "C" int64_t dflash_gguf_get_f64_array(const dflash_gguf *g, const char *key, double *out, int64_t cap) {
    const Value *v = find_kv(g, key);
    if (!v) return -1;
    if (v->type != T_ARR || (v->item_type != T_F32 && v->item_type != T_F64)) return -2;
    const size_t sz = scalar_size(v->item_type);
    for (uint64_t i = 0; i < v->len && out && static_cast<int64_t>(i) < cap; i++) float_as_f64(g, v->item_type, v->at + i * sz, &out[i]);
    return static_cast<int64_t>(v->len);
}

// ---- drafter loader ------------------------------------------------------------------

namespace {

// Metadata keys and tensor names of the two drafter conventions (loader.rs:842-917).
struct DrafterKeys {
    const char *block_count, *embedding_length, *feed_forward_length, *head_count, *head_count_kv, *key_length, *freq_base,
        *rms_norm_eps, *causal, *sliding_window, *sliding_window_pattern, *block_size, *mask_token_id, *target_layer_ids,
        *n_target_features /* null: derived */, *fc_tensor, *hidden_norm_tensor, *post_attn_norm_suffix;
};
const DrafterKeys kV1 = {"dflash-draft.block_count", "dflash-draft.embedding_length", "dflash-draft.feed_forward_length",
                         "dflash-draft.attention.head_count", "dflash-draft.attention.head_count_kv",
                         "dflash-draft.attention.key_length", "dflash-draft.rope.freq_base",
                         "dflash-draft.attention.layer_norm_rms_epsilon", "dflash-draft.attention.causal",
                         "dflash-draft.attention.sliding_window", "dflash-draft.attention.sliding_window_pattern",
                         "dflash-draft.dflash.block_size", "dflash-draft.dflash.mask_token_id",
                         "dflash-draft.dflash.target_layer_ids", "dflash-draft.dflash.n_target_features", "dflash_fc.weight",
                         "dflash_hidden_norm.weight", "post_attention_norm"};
const DrafterKeys kV2 = {"dflash.block_count", "dflash.embedding_length", "dflash.feed_forward_length",
                         "dflash.attention.head_count", "dflash.attention.head_count_kv", "dflash.attention.key_length",
                         "dflash.rope.freq_base", "dflash.attention.layer_norm_rms_epsilon", "dflash.attention.causal",
                         "dflash.attention.sliding_window", "dflash.attention.sliding_window_pattern", "dflash.block_size",
                         "tokenizer.ggml.mask_token_id", "dflash.target_layers", nullptr, "fc.weight",
                         "enc.output_norm.weight", "ffn_norm"};

struct Loader {
    dflash_gguf *g;
    int32_t rc = DFLASH_OK;

    bool bad(const char *what) {
        if (!rc) rc = fail(g, DFLASH_ERR_METADATA, "bad or missing metadata: %s", what);
        return false;
    }
    // required integer key that fits u32 (u64_to_u32, loader.rs)
    bool u32_key(const char *key, uint32_t *out) {
        uint64_t v = 0;
        if (!dflash_gguf_get_u64(g, key, &v)) return bad(key);
        if (v > 0xFFFFFFFFull) {
            if (!rc) rc = fail(g, DFLASH_ERR_METADATA, "metadata %s = %llu does not fit 32 bits", key, static_cast<unsigned long long>(v));
            return false;
        }
        *out = static_cast<uint32_t>(v);
        return true;
    }
    bool in_range(const char *key, uint64_t v, uint64_t cap) {
        if (v == 0) {
            if (!rc) rc = fail(g, DFLASH_ERR_METADATA, "metadata %s must be nonzero", key);
            return false;
        }
        if (v > cap) {
            if (!rc) rc = fail(g, DFLASH_ERR_METADATA, "metadata %s = %llu exceeds the cap %llu", key, static_cast<unsigned long long>(v), static_cast<unsigned long long>(cap));
            return false;
        }
        return true;
    }
    // need + check_shape (loader.rs:1292-1312); f32_only: the kernels read these as f32 vectors
    bool tensor(const std::string &name, std::initializer_list<uint64_t> shape, dflash_gguf_tensor *out, bool f32_only = false) {
        if (rc) return false;
        if (!dflash_gguf_find(g, name.c_str(), out)) {
            rc = fail(g, DFLASH_ERR_METADATA, "missing tensor %s", name.c_str());
            return false;
        }
        // trailing 1s of the expectation are not dimensions either
        std::vector<uint64_t> want(shape);
        while (want.size() > 1 && want.back() == 1) want.pop_back();
        bool same = static_cast<size_t>(out->n_dims) == want.size();
        for (size_t i = 0; same && i < want.size(); i++) same = out->shape[i] == want[i];
        if (!same) {
            std::string w, got;
            for (uint64_t d : want) w += (w.empty() ? "" : ", ") + std::to_string(d);
            for (int i = 0; i < out->n_dims; i++) got += (got.empty() ? "" : ", ") + std::to_string(out->shape[i]);
            rc = fail(g, DFLASH_ERR_METADATA, "tensor %s: expected shape [%s], got [%s]", name.c_str(), w.c_str(), got.c_str());
            return false;
        }
        if (f32_only && out->type != DFLASH_TYPE_F32) {
            rc = fail(g, DFLASH_ERR_UNSUPPORTED, "tensor %s must be F32 (type %d)", name.c_str(), out->type);
            return false;
        }
        return true;
    }
};

}  // namespace

static int32_t open_drafter_impl(dflash_gguf *g, const dflash_target_shape *target, dflash_gguf_draft_head *out,
                                 dflash_gguf_draft_layer *layers, int32_t layer_cap) {
    if (!g) return DFLASH_ERR_INVALID_INPUT;
    if (!target || !out || !layers) return fail(g, DFLASH_ERR_INVALID_INPUT, "open_drafter: null argument");
    if (target->hidden_size == 0 || target->vocab_size == 0 || target->n_layer == 0)
        return fail(g, DFLASH_ERR_METADATA, "DFlash target dimensions must be nonzero");
    memset(out, 0, sizeof(*out));
    const char *arch = nullptr;
    uint64_t arch_len = 0;
    const bool has_arch = dflash_gguf_get_str(g, "general.architecture", &arch, &arch_len) != 0;
    const std::string arch_s = has_arch ? std::string(arch, arch_len) : std::string();
    const DrafterKeys *k = nullptr;
    if (arch_s == "dflash-draft") k = &kV1;
    else if (arch_s == "dflash") k = &kV2;
    else return fail(g, DFLASH_ERR_METADATA, "unsupported architecture \"%s\" (a drafter is dflash-draft or dflash)", arch_s.c_str());
    out->convention = k == &kV1 ? 1 : 2;

    Loader L{g};
    uint32_t n_layer = 0, hidden = 0, ffn = 0, n_q = 0, n_kv = 0, head_dim = 0, block_size = 0;
    if (!L.u32_key(k->block_count, &n_layer) || !L.u32_key(k->embedding_length, &hidden) ||
        !L.u32_key(k->feed_forward_length, &ffn) || !L.u32_key(k->head_count, &n_q) || !L.u32_key(k->head_count_kv, &n_kv) ||
        !L.u32_key(k->key_length, &head_dim))
        return L.rc;
    double theta = 10000000.0;  // the loader's default when rope.freq_base is absent (loader.rs:956)
    dflash_gguf_get_f64(g, k->freq_base, &theta);
    double eps = 1e-6;
    if (find_kv(g, k->rms_norm_eps) && !dflash_gguf_get_f64(g, k->rms_norm_eps, &eps)) return L.bad(k->rms_norm_eps), L.rc;
    if (!(eps > 0.0) || !(eps <= 3.4028234663852886e38) || static_cast<float>(eps) == 0.0f) return L.bad(k->rms_norm_eps), L.rc;
    int32_t causal = 1;
    if (find_kv(g, k->causal) && !dflash_gguf_get_bool(g, k->causal, &causal)) return L.bad(k->causal), L.rc;
    uint32_t swa_window = 0;
    {
        uint64_t v = 0;
        if (dflash_gguf_get_u64(g, k->sliding_window, &v)) {
            if (v > 0xFFFFFFFFull) return L.bad(k->sliding_window), L.rc;
            swa_window = static_cast<uint32_t>(v);
        }
    }
    if (!L.u32_key(k->block_size, &block_size)) return L.rc;
    uint64_t mask = 0;
    if (!dflash_gguf_get_u64(g, k->mask_token_id, &mask) || mask > 0x7FFFFFFFull || mask >= target->vocab_size)
        return L.bad(k->mask_token_id), L.rc;
    out->mask_token_id = static_cast<int32_t>(mask);

    uint64_t ids[DFLASH_GGUF_MAX_TAPS];
    const int64_t n_ids = dflash_gguf_get_u64_array(g, k->target_layer_ids, ids, DFLASH_GGUF_MAX_TAPS);
    if (n_ids < 0) return L.bad(k->target_layer_ids), L.rc;
    if (n_ids == 0 || n_ids > DFLASH_GGUF_MAX_TAPS)
        return fail(g, DFLASH_ERR_METADATA, "metadata %s: %lld tapped layers (1..%d supported)", k->target_layer_ids, static_cast<long long>(n_ids), DFLASH_GGUF_MAX_TAPS);
    for (int64_t i = 0; i < n_ids; i++)
        if (ids[i] > 0xFFFFFFFFull) return L.bad(k->target_layer_ids), L.rc;
    uint64_t n_feat = static_cast<uint64_t>(n_ids) * target->hidden_size;
    if (k->n_target_features) {
        uint32_t v = 0;
        if (!L.u32_key(k->n_target_features, &v)) return L.rc;
        n_feat = v;
    } else if (n_feat > 0xFFFFFFFFull) {
        return L.bad(k->target_layer_ids), L.rc;
    }
    uint8_t pattern[kMaxArchLayers];
    const int64_t n_pattern = dflash_gguf_get_bool_array(g, k->sliding_window_pattern, pattern, kMaxArchLayers);
    if (n_pattern < 0) return L.bad(k->sliding_window_pattern), L.rc;
    // the "dflash" convention stores layer-input indices (post-block index + 1)
    if (out->convention == 2)
        for (int64_t i = 0; i < n_ids; i++) {
            if (ids[i] == 0)
                return fail(g, DFLASH_ERR_METADATA, "dflash.target_layers cannot capture layer input 0 as a post-block state");
            ids[i] -= 1;
        }

    // DFlash-2: presence of selector_hidden.weight makes the conv / selector metadata and tensors mandatory
    const bool v2 = dflash_gguf_find(g, "selector_hidden.weight", nullptr) != 0;
    uint32_t ck = 0, cg = 0, rank = 0, top_k = 0;
    if (v2) {
        if (!L.u32_key("dflash.conv_kernel_size", &ck) || !L.u32_key("dflash.conv_group_size", &cg) ||
            !L.u32_key("dflash.selector_rank", &rank) || !L.u32_key("dflash.selector_top_k", &top_k))
            return L.rc;
        if (!L.in_range("dflash.conv_kernel_size", ck, 8) || !L.in_range("dflash.conv_group_size", cg, 0xFFFFFFFFull) ||
            !L.in_range("dflash.selector_rank", rank, kMaxArchDim) || !L.in_range("dflash.selector_top_k", top_k, 64))
            return L.rc;
        if (hidden % cg) return fail(g, DFLASH_ERR_METADATA, "dflash.conv_group_size must divide embedding_length");
    }

    if (!L.in_range(k->block_count, n_layer, kMaxArchLayers) || !L.in_range(k->embedding_length, hidden, kMaxArchDim) ||
        !L.in_range(k->feed_forward_length, ffn, kMaxArchDim) || !L.in_range(k->head_count, n_q, kMaxArchDim) ||
        !L.in_range(k->head_count_kv, n_kv, kMaxArchDim))
        return L.rc;
    if (n_q % n_kv) return fail(g, DFLASH_ERR_METADATA, "%s (%u) must be a multiple of %s (%u)", k->head_count, n_q, k->head_count_kv, n_kv);
    if (!L.in_range(k->key_length, head_dim, kMaxArchDim) || !L.in_range(k->block_size, block_size, kMaxBlockSize) ||
        !L.in_range("n_target_features", n_feat, kMaxArchDim))
        return L.rc;
    if (hidden != target->hidden_size)
        return fail(g, DFLASH_ERR_METADATA, "%s (%u) must equal the target's hidden size (%u): the drafter shares the target's embedding and output head", k->embedding_length, hidden, target->hidden_size);
    if (n_feat != static_cast<uint64_t>(n_ids) * target->hidden_size)
        return fail(g, DFLASH_ERR_METADATA, "n_target_features mismatch: expected tapped layers x target hidden = %llu, got %llu", static_cast<unsigned long long>(static_cast<uint64_t>(n_ids) * target->hidden_size), static_cast<unsigned long long>(n_feat));
    for (int64_t i = 0; i < n_ids; i++)
        if (ids[i] >= target->n_layer)
            return fail(g, DFLASH_ERR_METADATA, "%s references layer %llu past the target's %u layers", k->target_layer_ids, static_cast<unsigned long long>(ids[i]), target->n_layer);
    if (n_pattern != static_cast<int64_t>(n_layer))
        return fail(g, DFLASH_ERR_METADATA, "%s length (%lld) must equal block_count (%u)", k->sliding_window_pattern, static_cast<long long>(n_pattern), n_layer);
    bool any_swa = false;
    for (uint32_t i = 0; i < n_layer; i++) any_swa |= pattern[i] != 0;
    if (swa_window == 0 && any_swa)
        return fail(g, DFLASH_ERR_METADATA, "drafter declares sliding-window layers but attention.sliding_window is missing or 0");
    const uint64_t q_dim = static_cast<uint64_t>(n_q) * head_dim, kv_dim = static_cast<uint64_t>(n_kv) * head_dim;
    if (q_dim > kMaxKernelDim || kv_dim > kMaxKernelDim) return fail(g, DFLASH_ERR_METADATA, "attention width exceeds %llu", static_cast<unsigned long long>(kMaxKernelDim));
    if (static_cast<int32_t>(n_layer) > layer_cap)
        return fail(g, DFLASH_ERR_INVALID_INPUT, "open_drafter: %u layers, room for %d", n_layer, layer_cap);

    dflash_draft_cfg &c = out->cfg;
    c.n_layers = static_cast<int32_t>(n_layer);
    c.hidden = static_cast<int32_t>(hidden);
    c.n_q = static_cast<int32_t>(n_q);
    c.n_kv = static_cast<int32_t>(n_kv);
    c.head_dim = static_cast<int32_t>(head_dim);
    c.ffn = static_cast<int32_t>(ffn);
    c.block_size = static_cast<int32_t>(block_size);
    c.n_taps = static_cast<int32_t>(n_ids);
    c.causal = causal;
    c.swa_window = swa_window;
    c.eps = static_cast<float>(eps);
    c.rope_theta = static_cast<float>(theta);
    c.conv_kernel_size = static_cast<int32_t>(ck);
    c.conv_group_size = static_cast<int32_t>(cg);
    c.selector_rank = static_cast<int32_t>(rank);
    c.selector_top_k = static_cast<int32_t>(top_k);
    out->n_target_layers = static_cast<int32_t>(n_ids);
    for (int64_t i = 0; i < n_ids; i++) out->target_layer_ids[i] = static_cast<int32_t>(ids[i]);

    const uint64_t h = hidden, f = ffn;
    L.tensor(k->fc_tensor, {n_feat, h}, &out->fc);
    L.tensor(k->hidden_norm_tensor, {h}, &out->hidden_norm, true);
    L.tensor("output_norm.weight", {h}, &out->output_norm, true);
    if (v2) {
        L.tensor("selector_predecessor.weight", {rank, target->vocab_size}, &out->selector_predecessor);
        L.tensor("selector_successor.weight", {rank, target->vocab_size}, &out->selector_successor);
        L.tensor("selector_hidden.weight", {h, rank}, &out->selector_hidden);
    }
    for (uint32_t i = 0; i < n_layer && !L.rc; i++) {
        dflash_gguf_draft_layer &Y = layers[i];
        memset(&Y, 0, sizeof(Y));
        const std::string b = "blk." + std::to_string(i) + ".";
        L.tensor(b + "attn_norm.weight", {h}, &Y.attn_norm, true);
        L.tensor(b + "attn_q.weight", {h, q_dim}, &Y.wq);
        L.tensor(b + "attn_k.weight", {h, kv_dim}, &Y.wk);
        L.tensor(b + "attn_v.weight", {h, kv_dim}, &Y.wv);
        L.tensor(b + "attn_output.weight", {q_dim, h}, &Y.wo);
        L.tensor(b + "attn_q_norm.weight", {head_dim}, &Y.q_norm, true);
        L.tensor(b + "attn_k_norm.weight", {head_dim}, &Y.k_norm, true);
        L.tensor(b + k->post_attn_norm_suffix + ".weight", {h}, &Y.post_norm, true);
        L.tensor(b + "ffn_gate.weight", {h, f}, &Y.gate);
        L.tensor(b + "ffn_up.weight", {h, f}, &Y.up);
        L.tensor(b + "ffn_down.weight", {f, h}, &Y.down);
        if (v2) {
            const uint64_t proj_out = 2ull * ck * (hidden / cg);
            L.tensor(b + "attn_conv_base", {h, ck, 2}, &Y.conv_attn_base, true);
            L.tensor(b + "attn_conv_proj.weight", {h, proj_out}, &Y.conv_attn_proj);
            L.tensor(b + "ffn_conv_base", {h, ck, 2}, &Y.conv_ffn_base, true);
            L.tensor(b + "ffn_conv_proj.weight", {h, proj_out}, &Y.conv_ffn_proj);
        }
        Y.is_swa = pattern[i] != 0;
    }
    return L.rc;
}

extern "C" int32_t dflash_gguf_open_drafter(dflash_gguf *g, const dflash_target_shape *target, dflash_gguf_draft_head *out,
                                            dflash_gguf_draft_layer *layers, int32_t layer_cap) {
    try {
        return open_drafter_impl(g, target, out, layers, layer_cap);
    } catch (const std::exception &e) {  // nothing may cross the C boundary
        return g ? fail(g, DFLASH_ERR_IO, "open_drafter: %s", e.what()) : DFLASH_ERR_IO;
    }
}
