// GGUF v3 reader and tensor upload: the file side of the quantized matmul path.
//
// Mirrors what the reference's loader accepts and rejects (src/loader/gguf/reader.rs:38-187:
// magic, version 3 only, key/value metadata, tensor infos, `general.alignment` with the
// default 32, data offset = aligned end of the infos, every tensor inside the file, no
// duplicate names; tensor bytes = ceil(ne0 / block) * block_bytes * ne1 * ...,
// src/loader/gguf/types.rs:443-472) and hands tensors over in the order the reference gives
// to its consumers: dimensions reversed to outermost-first (reader.rs:593-598).  The file is
// mapped read-only; tensor data is never copied on the host, uploads go straight from the
// mapping to device memory.
#include "gq_host_internal.h"

#include <hip/hip_runtime_api.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace {

constexpr uint32_t kMagic = 0x46554747u; // "GGUF"
constexpr uint32_t kVersion = 3;

// GgmlDType ids with their block geometry (src/loader/gguf/types.rs:57-94,152-236)
struct DType { uint32_t id, block_size, block_bytes; };
const DType kDTypes[] = {
    { 0, 1, 4 },      { 1, 1, 2 },      { 2, 32, 18 },    { 3, 32, 20 },    { 6, 32, 22 },    { 7, 32, 24 },
    { 8, 32, 34 },    { 9, 32, 36 },    { 10, 256, 84 },  { 11, 256, 110 }, { 12, 256, 144 }, { 13, 256, 176 },
    { 14, 256, 210 }, { 15, 256, 292 }, { 16, 256, 66 },  { 17, 256, 74 },  { 18, 256, 98 },  { 19, 256, 50 },
    { 20, 32, 18 },   { 21, 256, 110 }, { 22, 256, 82 },  { 23, 256, 136 }, { 24, 1, 1 },     { 25, 1, 2 },
    { 26, 1, 4 },     { 27, 1, 8 },     { 28, 1, 8 },     { 29, 256, 56 },  { 30, 1, 2 },     { 34, 256, 54 },
    { 35, 256, 66 },  { 39, 32, 17 },   { 50, 128, 72 },  { 51, 128, 72 },  { 52, 256, 130 }, { 53, 64, 36 },
};
const DType *find_dtype(uint32_t id)
{
    for (const DType &d : kDTypes)
        if (d.id == id) return &d;
    return nullptr;
}

struct Value {
    uint32_t type = 0;      // GgufValueType 0..12
    uint64_t bits = 0;      // scalars: the raw little-endian value, zero-extended
    const char *str = nullptr; // strings: bytes inside the file image
    uint64_t len = 0;       // strings: byte length; arrays: element count
    uint32_t item_type = 0; // arrays
    size_t items_at = 0;    // arrays: file position of the first element
};

struct Tensor {
    std::string name;
    uint32_t dtype = 0, n_dims = 0;
    uint64_t ne[4] = { 0, 0, 0, 0 }; // file order: ne[0] innermost
    size_t offset = 0, nbytes = 0;   // absolute position in the file
};

struct Error {
    int code = GLLMQ_GGUF_OK;
    std::string msg;
};

} // namespace

struct gllmq_gguf {
    const uint8_t *bytes = nullptr;
    size_t len = 0;
    bool mapped = false;
    uint32_t version = 0;
    uint64_t tensor_count = 0, kv_count = 0;
    size_t alignment = 32, data_offset = 0;
    std::map<std::string, Value> meta;
    std::vector<Tensor> tensors;
    std::map<std::string, size_t> index;
    // layer -> (projection -> tensor index) over the per-layer weights "blk.{layer}.{projection}.weight",
    // built once when the file is opened; layers at or beyond `layer_limit` are not in it
    std::map<size_t, std::map<std::string, size_t>> layers;
    size_t layer_limit = 0;
};

namespace {

// Well-formed UTF-8 as Rust's str::from_utf8 defines it (the reference reads every string
// through it): no overlong forms, no surrogates, nothing above U+10FFFF.
bool valid_utf8(const uint8_t *s, size_t n)
{
    size_t i = 0;
    while (i < n) {
        const uint8_t c = s[i];
        size_t need;
        uint32_t lo, hi = 0xBF;
        if (c < 0x80) { ++i; continue; }
        if (c >= 0xC2 && c <= 0xDF) { need = 1; lo = 0x80; }
        else if (c == 0xE0) { need = 2; lo = 0xA0; }
        else if (c >= 0xE1 && c <= 0xEC) { need = 2; lo = 0x80; }
        else if (c == 0xED) { need = 2; lo = 0x80; hi = 0x9F; }
        else if (c >= 0xEE && c <= 0xEF) { need = 2; lo = 0x80; }
        else if (c == 0xF0) { need = 3; lo = 0x90; }
        else if (c >= 0xF1 && c <= 0xF3) { need = 3; lo = 0x80; }
        else if (c == 0xF4) { need = 3; lo = 0x80; hi = 0x8F; }
        else return false;
        if (n - i <= need) return false;
        if (s[i + 1] < lo || s[i + 1] > hi) return false;
        for (size_t j = 2; j <= need; ++j)
            if ((s[i + j] & 0xC0) != 0x80) return false;
        i += need + 1;
    }
    return true;
}

struct Cursor {
    const uint8_t *p;
    size_t len, pos = 0;
    Error err;

    bool fail(int code, const char *fmt, ...)
    {
        if (err.code != GLLMQ_GGUF_OK) return false;
        char buf[256];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        err.code = code;
        err.msg = buf;
        return false;
    }
    bool take(size_t n, const uint8_t **out)
    {
        if (n > len - pos) return fail(GLLMQ_GGUF_ERR_PARSE, "unexpected end of file at byte %zu", pos);
        *out = p + pos;
        pos += n;
        return true;
    }
    bool uint(size_t n, uint64_t *v)
    {
        const uint8_t *b;
        if (!take(n, &b)) return false;
        uint64_t r = 0;
        for (size_t i = 0; i < n; ++i) r |= static_cast<uint64_t>(b[i]) << (8 * i);
        *v = r;
        return true;
    }
    bool string(const char **s, uint64_t *n)
    {
        uint64_t l;
        if (!uint(8, &l)) return false;
        if (l > len - pos) return fail(GLLMQ_GGUF_ERR_PARSE, "unexpected end of file in a string of %llu bytes",
                                       static_cast<unsigned long long>(l));
        if (!valid_utf8(p + pos, static_cast<size_t>(l))) return fail(GLLMQ_GGUF_ERR_UTF8, "a string at byte %zu is not UTF-8", pos);
        *s = reinterpret_cast<const char *>(p + pos);
        *n = l;
        pos += static_cast<size_t>(l);
        return true;
    }
};

size_t scalar_bytes(uint32_t type)
{
    switch (type) {
    case 0: case 1: case 7: return 1;
    case 2: case 3: return 2;
    case 4: case 5: case 6: return 4;
    case 10: case 11: case 12: return 8;
    default: return 0;
    }
}

// One metadata value at the cursor; arrays are walked (to find their end) but kept as a
// position, nested arrays included.
bool parse_value(Cursor &c, uint32_t type, Value *v, int depth)
{
    v->type = type;
    if (type > 12) return c.fail(GLLMQ_GGUF_ERR_PARSE, "unknown metadata value type %u", type);
    if (type == 8) return c.string(&v->str, &v->len);
    if (type == 9) {
        uint64_t it, n;
        if (!c.uint(4, &it) || !c.uint(8, &n)) return false;
        if (it > 12) return c.fail(GLLMQ_GGUF_ERR_PARSE, "unknown array item type %llu", static_cast<unsigned long long>(it));
        if (depth > 8) return c.fail(GLLMQ_GGUF_ERR_PARSE, "arrays nested too deeply");
        v->item_type = static_cast<uint32_t>(it);
        v->len = n;
        v->items_at = c.pos;
        const size_t sb = scalar_bytes(v->item_type);
        if (sb) { // fixed-size items: one bounds check
            if (n > (c.len - c.pos) / sb) return c.fail(GLLMQ_GGUF_ERR_PARSE, "unexpected end of file in an array");
            c.pos += static_cast<size_t>(n) * sb;
            return true;
        }
        for (uint64_t i = 0; i < n; ++i) {
            Value item;
            if (!parse_value(c, v->item_type, &item, depth + 1)) return false;
        }
        return true;
    }
    return c.uint(scalar_bytes(type), &v->bits);
}

// Value::as_u64 of the reference: unsigned kinds as they are, signed kinds when not negative
bool as_u64(const Value &v, uint64_t *out)
{
    switch (v.type) {
    case 0: case 2: case 4: case 10: *out = v.bits; return true;
    case 1: { const int8_t s = static_cast<int8_t>(v.bits); if (s < 0) return false; *out = static_cast<uint64_t>(s); return true; }
    case 3: { const int16_t s = static_cast<int16_t>(v.bits); if (s < 0) return false; *out = static_cast<uint64_t>(s); return true; }
    case 5: { const int32_t s = static_cast<int32_t>(v.bits); if (s < 0) return false; *out = static_cast<uint64_t>(s); return true; }
    case 11: { const int64_t s = static_cast<int64_t>(v.bits); if (s < 0) return false; *out = static_cast<uint64_t>(s); return true; }
    default: return false;
    }
}

bool mul_overflow(size_t a, size_t b, size_t *r) { return __builtin_mul_overflow(a, b, r); }

bool parse(gllmq_gguf *g, Error *err)
{
    Cursor c{ g->bytes, g->len, 0, {} };
    uint64_t v;
    if (!c.uint(4, &v)) { *err = c.err; return false; }
    if (v != kMagic) {
        err->code = GLLMQ_GGUF_ERR_MAGIC;
        char b[64];
        snprintf(b, sizeof b, "invalid magic 0x%08llx", static_cast<unsigned long long>(v));
        err->msg = b;
        return false;
    }
    if (!c.uint(4, &v)) { *err = c.err; return false; }
    g->version = static_cast<uint32_t>(v);
    if (g->version != kVersion) {
        err->code = GLLMQ_GGUF_ERR_VERSION;
        err->msg = "unsupported GGUF version " + std::to_string(g->version) + " (3 is read)";
        return false;
    }
    if (!c.uint(8, &g->tensor_count) || !c.uint(8, &g->kv_count)) { *err = c.err; return false; }
    // every key/value pair and every tensor info takes more than 8 bytes of file
    if (g->kv_count > g->len / 8 || g->tensor_count > g->len / 8) {
        err->code = GLLMQ_GGUF_ERR_PARSE;
        err->msg = "tensor or metadata count exceeds what the file can hold";
        return false;
    }
    for (uint64_t i = 0; i < g->kv_count; ++i) {
        const char *k;
        uint64_t kl, type;
        Value val;
        if (!c.string(&k, &kl) || !c.uint(4, &type) || !parse_value(c, static_cast<uint32_t>(type), &val, 0)) {
            *err = c.err;
            return false;
        }
        g->meta[std::string(k, static_cast<size_t>(kl))] = val; // a repeated key keeps the later value
    }
    struct Raw { Tensor t; uint64_t rel; };
    std::vector<Raw> raw;
    raw.reserve(static_cast<size_t>(g->tensor_count));
    for (uint64_t i = 0; i < g->tensor_count; ++i) {
        Raw r;
        const char *n;
        uint64_t nl, nd, dt;
        if (!c.string(&n, &nl) || !c.uint(4, &nd)) { *err = c.err; return false; }
        r.t.name.assign(n, static_cast<size_t>(nl));
        if (nd > 4) {
            c.fail(GLLMQ_GGUF_ERR_PARSE, "tensor %s has %llu dimensions (at most 4 are read)", r.t.name.c_str(),
                   static_cast<unsigned long long>(nd));
            *err = c.err;
            return false;
        }
        r.t.n_dims = static_cast<uint32_t>(nd);
        for (uint32_t d = 0; d < r.t.n_dims; ++d)
            if (!c.uint(8, &r.t.ne[d])) { *err = c.err; return false; }
        if (!c.uint(4, &dt) || !c.uint(8, &r.rel)) { *err = c.err; return false; }
        r.t.dtype = static_cast<uint32_t>(dt);
        if (!find_dtype(r.t.dtype)) {
            c.fail(GLLMQ_GGUF_ERR_DTYPE, "tensor %s has unknown ggml dtype %u", r.t.name.c_str(), r.t.dtype);
            *err = c.err;
            return false;
        }
        raw.push_back(std::move(r));
    }
    uint64_t al = 32;
    const auto it = g->meta.find("general.alignment");
    if (it != g->meta.end() && !as_u64(it->second, &al)) al = 32; // not an unsigned number: the default, as the reference
    if (al == 0) {
        err->code = GLLMQ_GGUF_ERR_METADATA;
        err->msg = "general.alignment must be > 0";
        return false;
    }
    if (al > g->len + 1) al = g->len + 1; // keeps the sum below in range; such a file has no room for data anyway
    g->alignment = static_cast<size_t>(al);
    g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    if (g->data_offset > g->len) {
        err->code = GLLMQ_GGUF_ERR_PARSE;
        err->msg = "tensor data offset exceeds file size";
        return false;
    }
    for (Raw &r : raw) {
        Tensor &t = r.t;
        const DType *d = find_dtype(t.dtype);
        size_t total = 0;
        if (t.n_dims > 0) { // rows are padded to whole blocks (types.rs:443-472)
            const uint64_t blocks = t.ne[0] / d->block_size + (t.ne[0] % d->block_size ? 1 : 0);
            bool over = blocks > SIZE_MAX / d->block_bytes;
            total = static_cast<size_t>(blocks) * d->block_bytes;
            for (uint32_t i = 1; i < t.n_dims && !over; ++i)
                over = t.ne[i] > SIZE_MAX || mul_overflow(total, static_cast<size_t>(t.ne[i]), &total);
            if (over) {
                err->code = GLLMQ_GGUF_ERR_PARSE;
                err->msg = "tensor byte size overflow: " + t.name;
                return false;
            }
        }
        t.nbytes = total;
        if (r.rel > g->len - g->data_offset || total > g->len - g->data_offset - static_cast<size_t>(r.rel)) {
            err->code = GLLMQ_GGUF_ERR_BOUNDS;
            err->msg = t.name + " lies beyond the end of the file";
            return false;
        }
        t.offset = g->data_offset + static_cast<size_t>(r.rel);
        if (!g->index.emplace(t.name, g->tensors.size()).second) {
            err->code = GLLMQ_GGUF_ERR_PARSE;
            err->msg = "duplicate tensor name: " + t.name;
            return false;
        }
        g->tensors.push_back(std::move(t));
    }
    return true;
}

void build_layer_table(gllmq_gguf *g);

int finish_open(gllmq_gguf *g, gllmq_gguf **out, char *err_buf, size_t err_len)
{
    Error e;
    if (parse(g, &e)) {
        build_layer_table(g);
        *out = g;
        return GLLMQ_GGUF_OK;
    }
    if (err_buf && err_len) snprintf(err_buf, err_len, "%s", e.msg.c_str());
    gllmq_gguf_close(g);
    return e.code;
}

// "blk.{layer}.{projection}.weight" -> (layer, projection); false for any other name
bool layer_weight_name(const std::string &name, size_t *layer, std::string *projection)
{
    if (name.compare(0, 4, "blk.") != 0) return false;
    const size_t dot1 = name.find('.', 4);
    if (dot1 == std::string::npos || dot1 == 4) return false;
    size_t l = 0;
    for (size_t i = 4; i < dot1; ++i) {
        if (name[i] < '0' || name[i] > '9' || l > (static_cast<size_t>(-1) >> 8)) return false;
        l = l * 10 + static_cast<size_t>(name[i] - '0');
    }
    const size_t dot2 = name.find('.', dot1 + 1);
    if (dot2 == std::string::npos || dot2 == dot1 + 1) return false;
    if (name.compare(dot2, std::string::npos, ".weight") != 0) return false;
    *layer = l;
    *projection = name.substr(dot1 + 1, dot2 - dot1 - 1);
    return true;
}

// The per-layer weights of the file.  Layer numbers come from tensor names, that is from the
// file: the table holds layers below the model's declared layer count ("{architecture}.block_count",
// when the file says so as an unsigned or non-negative number) and never more layers than the
// file has tensors, so a stray "blk.99999999999999.x.weight" costs nothing.  The reference groups
// layers below the model's num_layers and ignores stray higher indices the same way
// (build_graph.inc.rs:416-428).
void build_layer_table(gllmq_gguf *g)
{
    size_t limit = g->tensors.size();
    const auto arch = g->meta.find("general.architecture");
    if (arch != g->meta.end() && arch->second.type == 8 && arch->second.str) { // 8: string
        const auto count = g->meta.find(std::string(arch->second.str, static_cast<size_t>(arch->second.len)) + ".block_count");
        if (count != g->meta.end()) {
            const Value &v = count->second;
            const bool is_unsigned = v.type == 0 || v.type == 2 || v.type == 4 || v.type == 10; // u8, u16, u32, u64
            const bool is_signed = v.type == 1 || v.type == 3 || v.type == 5 || v.type == 11;   // i8, i16, i32, i64
            uint64_t n = v.bits;
            bool ok = is_unsigned;
            if (is_signed) {
                const int bits = v.type == 1 ? 8 : v.type == 3 ? 16 : v.type == 5 ? 32 : 64;
                ok = bits == 64 ? static_cast<int64_t>(n) >= 0 : ((n >> (bits - 1)) & 1u) == 0u;
            }
            if (ok && n < limit) limit = static_cast<size_t>(n);
        }
    }
    g->layer_limit = limit;
    for (size_t i = 0; i < g->tensors.size(); ++i) {
        size_t layer;
        std::string proj;
        if (layer_weight_name(g->tensors[i].name, &layer, &proj) && layer < limit) g->layers[layer][proj] = i;
    }
}

const Value *find_meta(const gllmq_gguf *g, const char *key)
{
    if (!g || !key) return nullptr;
    const auto it = g->meta.find(key);
    return it == g->meta.end() ? nullptr : &it->second;
}

} // namespace

extern "C" {

int gllmq_gguf_open(const char *path, gllmq_gguf **out, char *err, size_t err_len)
{
    if (!path || !out) return GLLMQ_GGUF_ERR_IO;
    *out = nullptr;
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (fd < 0 || fstat(fd, &st) != 0) {
        if (err && err_len) snprintf(err, err_len, "%s: %s", path, strerror(errno));
        if (fd >= 0) close(fd);
        return GLLMQ_GGUF_ERR_IO;
    }
    gllmq_gguf *g = new gllmq_gguf;
    g->len = static_cast<size_t>(st.st_size);
    if (g->len > 0) {
        void *m = mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (m == MAP_FAILED) {
            if (err && err_len) snprintf(err, err_len, "%s: mmap: %s", path, strerror(errno));
            close(fd);
            delete g;
            return GLLMQ_GGUF_ERR_IO;
        }
        g->bytes = static_cast<const uint8_t *>(m);
        g->mapped = true;
    }
    close(fd);
    return finish_open(g, out, err, err_len);
}

int gllmq_gguf_parse(const void *bytes, size_t len, gllmq_gguf **out, char *err, size_t err_len)
{
    if (!out || (!bytes && len)) return GLLMQ_GGUF_ERR_IO;
    *out = nullptr;
    gllmq_gguf *g = new gllmq_gguf;
    g->bytes = static_cast<const uint8_t *>(bytes);
    g->len = len;
    return finish_open(g, out, err, err_len);
}

void gllmq_gguf_close(gllmq_gguf *g)
{
    if (!g) return;
    if (g->mapped) munmap(const_cast<uint8_t *>(g->bytes), g->len);
    delete g;
}

uint32_t gllmq_gguf_version(const gllmq_gguf *g) { return g ? g->version : 0; }
size_t gllmq_gguf_tensor_count(const gllmq_gguf *g) { return g ? g->tensors.size() : 0; }
size_t gllmq_gguf_kv_count(const gllmq_gguf *g) { return g ? static_cast<size_t>(g->kv_count) : 0; }
size_t gllmq_gguf_alignment(const gllmq_gguf *g) { return g ? g->alignment : 0; }
size_t gllmq_gguf_data_offset(const gllmq_gguf *g) { return g ? g->data_offset : 0; }

int gllmq_gguf_tensor_at(const gllmq_gguf *g, size_t index, gllmq_gguf_tensor *out)
{
    if (!g || !out || index >= g->tensors.size()) return GLLMQ_GGUF_ERR_BOUNDS;
    const Tensor &t = g->tensors[index];
    out->name = t.name.c_str();
    out->ggml_dtype = t.dtype;
    out->n_dims = t.n_dims;
    for (uint32_t i = 0; i < 4; ++i) {
        out->ne[i] = i < t.n_dims ? t.ne[i] : 0;
        out->shape[i] = i < t.n_dims ? t.ne[t.n_dims - 1 - i] : 0; // outermost first
    }
    out->offset = t.offset;
    out->nbytes = t.nbytes;
    return GLLMQ_GGUF_OK;
}

long gllmq_gguf_find_tensor(const gllmq_gguf *g, const char *name)
{
    if (!g || !name) return -1;
    const auto it = g->index.find(name);
    return it == g->index.end() ? -1 : static_cast<long>(it->second);
}

const void *gllmq_gguf_tensor_data(const gllmq_gguf *g, size_t index)
{
    if (!g || index >= g->tensors.size()) return nullptr;
    return g->bytes + g->tensors[index].offset;
}

size_t gllmq_gguf_layer_count(const gllmq_gguf *g)
{
    if (!g) return 0;
    return g->layers.empty() ? 0 : g->layers.rbegin()->first + 1;
}

size_t gllmq_gguf_layer_tensors(const gllmq_gguf *g, size_t layer, size_t *indices, size_t capacity)
{
    if (!g) return 0;
    const auto &table = g->layers;
    const auto it = table.find(layer);
    if (it == table.end()) return 0;
    size_t n = 0;
    for (const auto &pt : it->second) { // projection-name order
        if (indices && n < capacity) indices[n] = pt.second;
        ++n;
    }
    return n;
}

long gllmq_gguf_layer_tensor(const gllmq_gguf *g, size_t layer, const char *projection)
{
    if (!g || !projection) return -1;
    const auto it = g->layers.find(layer);
    if (it == g->layers.end()) return -1;
    const auto pt = it->second.find(projection);
    return pt == it->second.end() ? -1 : static_cast<long>(pt->second);
}

size_t gllmq_gguf_mixed_quant_groups(const gllmq_gguf *g, uint32_t *group_of, size_t capacity)
{
    if (!g) return 0;
    const auto &table = g->layers;
    // a layer's signature: its (projection, dtype) pairs in projection order
    typedef std::vector<std::pair<std::string, uint32_t>> Signature;
    std::map<Signature, std::vector<size_t>> by_signature;
    for (const auto &lt : table) {
        Signature sig;
        for (const auto &pt : lt.second) sig.emplace_back(pt.first, g->tensors[pt.second].dtype);
        by_signature[sig].push_back(lt.first); // layers arrive in ascending order
    }
    for (size_t i = 0; group_of && i < capacity; ++i) group_of[i] = UINT32_MAX;
    if (by_signature.size() <= 1) return 0;
    // groups are numbered in signature order (pairs compared in turn, a prefix before its extensions)
    uint32_t gi = 0;
    for (const auto &sg : by_signature) {
        for (size_t layer : sg.second)
            if (group_of && layer < capacity) group_of[layer] = gi;
        ++gi;
    }
    return by_signature.size();
}

int gllmq_gguf_meta_type(const gllmq_gguf *g, const char *key)
{
    const Value *v = find_meta(g, key);
    return v ? static_cast<int>(v->type) : -1;
}

int gllmq_gguf_meta_u64(const gllmq_gguf *g, const char *key, uint64_t *out)
{
    const Value *v = find_meta(g, key);
    uint64_t r;
    if (!v || !out || !as_u64(*v, &r)) return 0;
    *out = r;
    return 1;
}

int gllmq_gguf_meta_i64(const gllmq_gguf *g, const char *key, int64_t *out)
{
    const Value *v = find_meta(g, key);
    if (!v || !out) return 0;
    switch (v->type) {
    case 0: case 2: case 4: *out = static_cast<int64_t>(v->bits); return 1;
    case 10: if (v->bits > static_cast<uint64_t>(INT64_MAX)) return 0; *out = static_cast<int64_t>(v->bits); return 1;
    case 1: *out = static_cast<int8_t>(v->bits); return 1;
    case 3: *out = static_cast<int16_t>(v->bits); return 1;
    case 5: *out = static_cast<int32_t>(v->bits); return 1;
    case 11: *out = static_cast<int64_t>(v->bits); return 1;
    default: return 0;
    }
}

int gllmq_gguf_meta_f64(const gllmq_gguf *g, const char *key, double *out)
{
    const Value *v = find_meta(g, key);
    if (!v || !out) return 0;
    if (v->type == 6) {
        float f;
        const uint32_t b = static_cast<uint32_t>(v->bits);
        memcpy(&f, &b, 4);
        *out = f;
        return 1;
    }
    if (v->type == 12) {
        memcpy(out, &v->bits, 8);
        return 1;
    }
    return 0;
}

int gllmq_gguf_meta_bool(const gllmq_gguf *g, const char *key, int *out)
{
    const Value *v = find_meta(g, key);
    if (!v || !out || v->type != 7) return 0;
    *out = v->bits != 0;
    return 1;
}

const char *gllmq_gguf_meta_str(const gllmq_gguf *g, const char *key, size_t *len)
{
    const Value *v = find_meta(g, key);
    if (!v || v->type != 8) return nullptr;
    if (len) *len = static_cast<size_t>(v->len);
    return v->str ? v->str : "";
}

int gllmq_gguf_meta_array(const gllmq_gguf *g, const char *key, uint32_t *item_type, uint64_t *count)
{
    const Value *v = find_meta(g, key);
    if (!v || v->type != 9) return 0;
    if (item_type) *item_type = v->item_type;
    if (count) *count = v->len;
    return 1;
}

const char *gllmq_gguf_meta_array_str(const gllmq_gguf *g, const char *key, uint64_t i, size_t *len)
{
    const Value *v = find_meta(g, key);
    if (!v || v->type != 9 || v->item_type != 8 || i >= v->len) return nullptr;
    Cursor c{ g->bytes, g->len, 0, {} };
    c.pos = v->items_at;
    const char *s = nullptr;
    uint64_t l = 0;
    for (uint64_t j = 0; j <= i; ++j)
        if (!c.string(&s, &l)) return nullptr;
    if (len) *len = static_cast<size_t>(l);
    return s;
}

int gllmq_gguf_upload(gllmq_ctx *ctx, const gllmq_gguf *g, size_t index, void *dst_dev, size_t dst_bytes, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    if (!g || index >= g->tensors.size() || !dst_dev) return gq_ctx_set_error(ctx, GLLMQ_ERR_INVALID, "gguf_upload: no such tensor or NULL destination");
    const Tensor &t = g->tensors[index];
    if (dst_bytes < t.nbytes)
        return gq_ctx_set_error(ctx, GLLMQ_ERR_BAD_SHAPE, "gguf_upload: destination too small for the tensor");
    if (t.nbytes == 0) return GLLMQ_OK;
    // pageable source: the runtime stages the copy and returns when the source has been read
    const hipError_t e = hipMemcpyAsync(dst_dev, g->bytes + t.offset, t.nbytes, hipMemcpyHostToDevice,
                                        static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return gq_ctx_set_error(ctx, GLLMQ_ERR_HIP, hipGetErrorString(e));
    return GLLMQ_OK;
}

} // extern "C"
