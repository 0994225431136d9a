// GGUF v3 container reader: the file side of the weight path.  Semantics follow the
// reference's src/gguf/mod.rs:97-217 (header, metadata, tensor directory, alignment,
// per-tensor bounds check), reader.rs:41-86 (little-endian cursor, length-prefixed UTF-8
// strings), tensor_info.rs:21-63 (1..4 dims, block-multiple element count) and
// types.rs:37-103 (type ids and block geometry).
//
// Built for a mapping, not for a parsed tree: the file is mmap'ed read-only and the
// directory keeps, per metadata entry, only the key, the value type and the OFFSET of
// the value in the mapping.  A tokenizer's 150k-string vocabulary costs one validating
// walk at open and no allocation; getters decode at the stored offset.  Tensor payloads
// are handed out as pointers into the mapping, which is what the repack routines read.
#include <cstring>
#include <fcntl.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

#include "../../../include/rein.h"
#include "hip_api.h"

namespace {

using rein::fail;

constexpr uint32_t kMagic = 0x46554747u;             // "GGUF"
constexpr uint32_t kVersion = 3;
constexpr uint64_t kDefaultAlignment = 32;
constexpr int kMaxArrayDepth = 4;

// gguf_metadata_value_type (types.rs:108-113)
enum : uint32_t { VT_U8, VT_I8, VT_U16, VT_I16, VT_U32, VT_I32, VT_F32, VT_BOOL, VT_STRING, VT_ARRAY, VT_U64, VT_I64, VT_F64, VT_END };

unsigned fixed_width(uint32_t vt)
{
    switch (vt) {
    case VT_U8: case VT_I8: case VT_BOOL: return 1;
    case VT_U16: case VT_I16: return 2;
    case VT_U32: case VT_I32: case VT_F32: return 4;
    case VT_U64: case VT_I64: case VT_F64: return 8;
    default: return 0;
    }
}

// weights per block / bytes per block of every tensor type the container may hold
// (types.rs:61-96); false for an id outside the table
bool ggml_geometry(uint32_t t, uint64_t* elems, uint64_t* bytes)
{
    struct G { uint32_t id; uint16_t e, b; };
    static const G tab[] = {{0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},   {6, 32, 22},   {7, 32, 24},
                            {8, 32, 34},    {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176},
                            {14, 256, 210}, {15, 256, 292}, {20, 32, 18},   {21, 256, 110}, {23, 256, 136}, {30, 1, 2}};
    for (const G& g : tab)
        if (g.id == t) { *elems = g.e; *bytes = g.b; return true; }
    return false;
}

bool utf8_ok(const uint8_t* s, size_t n)
{
    size_t i = 0;
    while (i < n) {
        const uint8_t c = s[i];
        if (c < 0x80) { i++; continue; }
        unsigned len;
        uint32_t cp;
        if ((c & 0xE0) == 0xC0) { len = 2; cp = c & 0x1Fu; }
        else if ((c & 0xF0) == 0xE0) { len = 3; cp = c & 0x0Fu; }
        else if ((c & 0xF8) == 0xF0) { len = 4; cp = c & 0x07u; }
        else return false;
        if (n - i < len) return false;
        for (unsigned k = 1; k < len; k++) {
            if ((s[i + k] & 0xC0) != 0x80) return false;
            cp = (cp << 6) | (s[i + k] & 0x3Fu);
        }
        static const uint32_t lowest[5] = {0, 0, 0x80, 0x800, 0x10000};
        if (cp < lowest[len] || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
        i += len;
    }
    return true;
}

struct Cursor {
    const uint8_t* buf;
    size_t len, pos;
    std::string err;

    bool need(size_t n)
    {
        if (len - pos >= n) return true;
        err = "truncated read: needed " + std::to_string(n) + " bytes at offset " + std::to_string(pos) + ", only " +
              std::to_string(len - pos) + " available";
        return false;
    }
    template <typename T> bool get(T* v)
    {
        if (!need(sizeof(T))) return false;
        std::memcpy(v, buf + pos, sizeof(T));             // the container is little-endian; so is every host this runs on
        pos += sizeof(T);
        return true;
    }
    // u64 length + bytes; returns the view
    bool str(const uint8_t** s, uint64_t* n)
    {
        const size_t at = pos;
        if (!get(n)) return false;
        if (*n > len - pos) { need(*n > (uint64_t)SIZE_MAX ? SIZE_MAX : (size_t)*n); return false; }
        *s = buf + pos;
        if (!utf8_ok(*s, (size_t)*n)) { err = "invalid UTF-8 in GGUF string at offset " + std::to_string(at); return false; }
        pos += (size_t)*n;
        return true;
    }
    // a key or tensor name: additionally free of NUL bytes, because the C ABI hands names
    // out and takes them in as NUL-terminated strings (the reference's String would hold one)
    bool name(const uint8_t** s, uint64_t* n)
    {
        const size_t at = pos;
        if (!str(s, n)) return false;
        if (std::memchr(*s, 0, (size_t)*n)) { err = "NUL byte in GGUF key or tensor name at offset " + std::to_string(at); return false; }
        return true;
    }
    // steps over one value of type vt, validating bounds, strings and nested types
    bool skip_value(uint32_t vt, int depth)
    {
        if (const unsigned w = fixed_width(vt)) {
            if (!need(w)) return false;
            pos += w;
            return true;
        }
        if (vt == VT_STRING) {
            const uint8_t* s;
            uint64_t n;
            return str(&s, &n);
        }
        if (vt != VT_ARRAY) { err = "unknown GGUF metadata value type: " + std::to_string(vt); return false; }
        if (depth >= kMaxArrayDepth) { err = "GGUF metadata arrays nested deeper than " + std::to_string(kMaxArrayDepth); return false; }
        uint32_t et;
        uint64_t n;
        if (!get(&et)) return false;
        if (et >= VT_END) { err = "unknown GGUF metadata value type: " + std::to_string(et); return false; }
        if (!get(&n)) return false;
        if (const unsigned w = fixed_width(et)) {
            if (n > (len - pos) / w) { need(SIZE_MAX); return false; }
            pos += (size_t)n * w;
            return true;
        }
        for (uint64_t i = 0; i < n; i++)
            if (!skip_value(et, depth + 1)) return false;
        return true;
    }
};

struct Meta {
    std::string key;
    uint32_t type;
    size_t value_at;          // offset of the value (for an array: of its element type word)
};

struct Tensor {
    std::string name;
    uint32_t type;
    uint32_t n_dims;
    uint64_t dims[4];
    uint64_t offset, byte_size;
};

}  // namespace

struct rein_gguf {
    const uint8_t* base = nullptr;
    size_t len = 0;
    bool mapped = false;
    uint32_t version = 0;
    uint64_t tensor_count = 0, kv_count = 0, alignment = 0, data_at = 0;
    std::vector<Meta> meta;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, size_t> meta_index, tensor_index;
};

namespace {

uint64_t align_up(uint64_t v, uint64_t a) { return a <= 1 ? v : (v + a - 1) / a * a; }

// byte size of a tensor from its shape and type (tensor_info.rs:34-46)
int tensor_byte_size(Tensor& t, std::string* err)
{
    uint64_t be, bb;
    if (!ggml_geometry(t.type, &be, &bb)) { *err = "unknown ggml tensor type: " + std::to_string(t.type); return REIN_E_BAD_FILE; }
    uint64_t n = 1;
    for (unsigned d = 0; d < t.n_dims; d++) {
        if (t.dims[d] != 0 && n > UINT64_MAX / t.dims[d]) {
            *err = "tensor `" + t.name + "` element count overflows 64 bits";
            return REIN_E_BAD_FILE;
        }
        n *= t.dims[d];
    }
    if (n % be != 0) {
        *err = "tensor `" + t.name + "` element count " + std::to_string(n) + " is not a multiple of block size " +
               std::to_string(be) + " for type " + std::to_string(t.type);
        return REIN_E_BAD_FILE;
    }
    if (n / be > UINT64_MAX / bb) { *err = "tensor `" + t.name + "` byte size overflows 64 bits"; return REIN_E_BAD_FILE; }
    t.byte_size = n / be * bb;
    return REIN_OK;
}

// GgufFile::from_mmap (mod.rs:104-177)
int parse(rein_gguf* g)
{
    Cursor c{g->base, g->len, 0, {}};
    uint32_t magic;
    if (!c.get(&magic)) return fail(REIN_E_BAD_FILE, c.err);
    if (magic != kMagic) {
        char hex[16];
        snprintf(hex, sizeof hex, "0x%08x", magic);
        return fail(REIN_E_BAD_FILE, std::string("not a GGUF file (bad magic: got ") + hex + ", expected 0x46554747 / \"GGUF\")");
    }
    if (!c.get(&g->version)) return fail(REIN_E_BAD_FILE, c.err);
    if (g->version != kVersion)
        return fail(REIN_E_BAD_FILE, "unsupported GGUF version: " + std::to_string(g->version) + " (only v3 is supported)");
    if (!c.get(&g->tensor_count) || !c.get(&g->kv_count)) return fail(REIN_E_BAD_FILE, c.err);

    for (uint64_t i = 0; i < g->kv_count; i++) {
        const uint8_t* s;
        uint64_t n;
        uint32_t vt;
        if (!c.name(&s, &n) || !c.get(&vt)) return fail(REIN_E_BAD_FILE, c.err);
        if (vt >= VT_END) return fail(REIN_E_BAD_FILE, "unknown GGUF metadata value type: " + std::to_string(vt));
        Meta m{std::string((const char*)s, (size_t)n), vt, c.pos};
        if (!c.skip_value(vt, 0)) return fail(REIN_E_BAD_FILE, c.err);
        g->meta_index[m.key] = g->meta.size();           // a repeated key resolves to its last entry
        g->meta.push_back(std::move(m));
    }
    for (uint64_t i = 0; i < g->tensor_count; i++) {
        const uint8_t* s;
        uint64_t n;
        Tensor t{};
        if (!c.name(&s, &n)) return fail(REIN_E_BAD_FILE, c.err);
        t.name.assign((const char*)s, (size_t)n);
        if (!c.get(&t.n_dims)) return fail(REIN_E_BAD_FILE, c.err);
        if (t.n_dims == 0 || t.n_dims > 4)
            return fail(REIN_E_BAD_FILE, "tensor `" + t.name + "` has invalid shape (n_dims=" + std::to_string(t.n_dims) +
                                             ", max 4 supported)");
        for (unsigned d = 0; d < 4; d++) t.dims[d] = 1;
        for (unsigned d = 0; d < t.n_dims; d++)
            if (!c.get(&t.dims[d])) return fail(REIN_E_BAD_FILE, c.err);
        if (!c.get(&t.type)) return fail(REIN_E_BAD_FILE, c.err);
        uint64_t be, bb;
        if (!ggml_geometry(t.type, &be, &bb)) return fail(REIN_E_BAD_FILE, "unknown ggml tensor type: " + std::to_string(t.type));
        if (!c.get(&t.offset)) return fail(REIN_E_BAD_FILE, c.err);
        g->tensor_index[t.name] = g->tensors.size();
        g->tensors.push_back(std::move(t));
    }

    g->alignment = kDefaultAlignment;
    uint64_t a;
    if (rein_gguf_meta_u64(g, "general.alignment", &a) == REIN_OK) g->alignment = a;
    if (c.pos > UINT64_MAX - g->alignment) return fail(REIN_E_BAD_FILE, "general.alignment out of range");
    g->data_at = align_up(c.pos, g->alignment);

    for (Tensor& t : g->tensors) {
        std::string err;
        if (int rc = tensor_byte_size(t, &err)) return fail(rc, err);
        if (t.offset > UINT64_MAX - g->data_at || t.byte_size > UINT64_MAX - g->data_at - t.offset ||
            g->data_at + t.offset + t.byte_size > g->len)
            return fail(REIN_E_BAD_FILE, "tensor `" + t.name + "` data extends past file end (offset=" +
                                             std::to_string(g->data_at + t.offset) + ", size=" + std::to_string(t.byte_size) +
                                             ", file_len=" + std::to_string(g->len) + ")");
    }
    return REIN_OK;
}

void fill(const rein_gguf* g, const Tensor& t, rein_gguf_tensor* out)
{
    out->name = t.name.c_str();
    out->ggml_type = (int)t.type;
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) out->dims[d] = t.dims[d];
    out->offset = t.offset;
    out->byte_size = t.byte_size;
    out->data = g->base + g->data_at + t.offset;
}

const Meta* find_meta(const rein_gguf* g, const char* key)
{
    if (!g || !key) return nullptr;
    auto it = g->meta_index.find(key);
    return it == g->meta_index.end() ? nullptr : &g->meta[it->second];
}

template <typename T> T load(const rein_gguf* g, size_t at)
{
    T v;
    std::memcpy(&v, g->base + at, sizeof(T));
    return v;
}

int not_found(const char* what, const char* name)
{
    return fail(REIN_E_NOT_FOUND, std::string(what) + " `" + (name ? name : "(null)") + "` not found");
}

}  // namespace

extern "C" {

uint64_t rein_gguf_align_up(uint64_t v, uint64_t align) { return align_up(v, align); }

int rein_gguf_from_bytes(const uint8_t* bytes, size_t len, rein_gguf** out)
{
    if (!out || (!bytes && len)) return fail(REIN_E_BAD_POINTER, "rein_gguf_from_bytes: null argument");
    *out = nullptr;
    rein_gguf* g = new rein_gguf;
    g->base = bytes;
    g->len = len;
    if (int rc = parse(g)) { delete g; return rc; }
    *out = g;
    return REIN_OK;
}

int rein_gguf_open(const char* path, rein_gguf** out)
{
    if (!path || !out) return fail(REIN_E_BAD_POINTER, "rein_gguf_open: null argument");
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail(REIN_E_BAD_FILE, std::string("io error: ") + path + ": " + std::strerror(errno));
    struct stat st;
    if (::fstat(fd, &st) != 0) {
        const int e = errno;
        ::close(fd);
        return fail(REIN_E_BAD_FILE, std::string("io error: ") + path + ": " + std::strerror(e));
    }
    rein_gguf* g = new rein_gguf;
    g->len = (size_t)st.st_size;
    if (g->len) {
        void* p = ::mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) {
            const int e = errno;
            ::close(fd);
            delete g;
            return fail(REIN_E_BAD_FILE, std::string("io error: mmap ") + path + ": " + std::strerror(e));
        }
        g->base = (const uint8_t*)p;
        g->mapped = true;
    }
    ::close(fd);                                          // the mapping outlives the descriptor
    if (int rc = parse(g)) { rein_gguf_close(g); return rc; }
    *out = g;
    return REIN_OK;
}

void rein_gguf_close(rein_gguf* g)
{
    if (!g) return;
    if (g->mapped) ::munmap(const_cast<uint8_t*>(g->base), g->len);
    delete g;
}

int rein_gguf_header(const rein_gguf* g, uint32_t* version, uint64_t* tensor_count, uint64_t* metadata_kv_count,
                     uint64_t* alignment, uint64_t* data_section_offset)
{
    if (!g) return fail(REIN_E_BAD_POINTER, "rein_gguf_header: null handle");
    if (version) *version = g->version;
    if (tensor_count) *tensor_count = g->tensor_count;
    if (metadata_kv_count) *metadata_kv_count = g->kv_count;
    if (alignment) *alignment = g->alignment;
    if (data_section_offset) *data_section_offset = g->data_at;
    return REIN_OK;
}

int rein_gguf_tensor_at(const rein_gguf* g, uint64_t index, rein_gguf_tensor* out)
{
    if (!g || !out) return fail(REIN_E_BAD_POINTER, "rein_gguf_tensor_at: null argument");
    if (index >= g->tensors.size()) return fail(REIN_E_NOT_FOUND, "tensor index " + std::to_string(index) + " out of range");
    fill(g, g->tensors[(size_t)index], out);
    return REIN_OK;
}

int rein_gguf_tensor_by_name(const rein_gguf* g, const char* name, rein_gguf_tensor* out)
{
    if (!g || !name || !out) return fail(REIN_E_BAD_POINTER, "rein_gguf_tensor_by_name: null argument");
    auto it = g->tensor_index.find(name);
    if (it == g->tensor_index.end()) return not_found("tensor", name);
    fill(g, g->tensors[it->second], out);
    return REIN_OK;
}

int rein_gguf_meta_at(const rein_gguf* g, uint64_t index, const char** key, int* value_type)
{
    if (!g) return fail(REIN_E_BAD_POINTER, "rein_gguf_meta_at: null handle");
    if (index >= g->meta.size()) return fail(REIN_E_NOT_FOUND, "metadata index " + std::to_string(index) + " out of range");
    if (key) *key = g->meta[(size_t)index].key.c_str();
    if (value_type) *value_type = (int)g->meta[(size_t)index].type;
    return REIN_OK;
}

int rein_gguf_meta_type(const rein_gguf* g, const char* key, int* value_type)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (value_type) *value_type = (int)m->type;
    return REIN_OK;
}

int rein_gguf_meta_raw(const rein_gguf* g, const char* key, int* value_type, const uint8_t** value)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (value_type) *value_type = (int)m->type;
    if (value) *value = g->base + m->value_at;
    return REIN_OK;
}

// MetaValue::as_u64 (value.rs:69-81): any integer variant that is non-negative
int rein_gguf_meta_u64(const rein_gguf* g, const char* key, uint64_t* out)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    int64_t s;
    switch (m->type) {
    case VT_U8:  *out = load<uint8_t>(g, m->value_at); return REIN_OK;
    case VT_U16: *out = load<uint16_t>(g, m->value_at); return REIN_OK;
    case VT_U32: *out = load<uint32_t>(g, m->value_at); return REIN_OK;
    case VT_U64: *out = load<uint64_t>(g, m->value_at); return REIN_OK;
    case VT_I8:  s = load<int8_t>(g, m->value_at); break;
    case VT_I16: s = load<int16_t>(g, m->value_at); break;
    case VT_I32: s = load<int32_t>(g, m->value_at); break;
    case VT_I64: s = load<int64_t>(g, m->value_at); break;
    default: return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is not an integer");
    }
    if (s < 0) return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is negative");
    *out = (uint64_t)s;
    return REIN_OK;
}

// MetaValue::as_f32 (value.rs:88-94); booleans are not numbers there either
int rein_gguf_meta_f32(const rein_gguf* g, const char* key, float* out)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (m->type == VT_F32) *out = load<float>(g, m->value_at);
    else if (m->type == VT_F64) *out = (float)load<double>(g, m->value_at);
    else return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is not a float");
    return REIN_OK;
}

int rein_gguf_meta_bool(const rein_gguf* g, const char* key, int* out)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (m->type != VT_BOOL) return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is not a bool");
    *out = load<uint8_t>(g, m->value_at) != 0;             // reader.rs:64-66
    return REIN_OK;
}

int rein_gguf_meta_str(const rein_gguf* g, const char* key, const char** s, size_t* len)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (m->type != VT_STRING) return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is not a string");
    *len = (size_t)load<uint64_t>(g, m->value_at);
    *s = (const char*)g->base + m->value_at + 8;           // not NUL-terminated
    return REIN_OK;
}

int rein_gguf_meta_array(const rein_gguf* g, const char* key, int* elem_type, uint64_t* count, const uint8_t** first)
{
    const Meta* m = find_meta(g, key);
    if (!m) return not_found("metadata key", key);
    if (m->type != VT_ARRAY) return fail(REIN_E_BAD_FORMAT, std::string("metadata key `") + key + "` is not an array");
    if (elem_type) *elem_type = (int)load<uint32_t>(g, m->value_at);
    if (count) *count = load<uint64_t>(g, m->value_at + 4);
    if (first) *first = g->base + m->value_at + 12;
    return REIN_OK;
}

// GpuMatvecTensor::from_gguf_matvec (src/runtime/qwen35.rs:235-245) and
// GpuExpertTensor::from_gguf (qwen35.rs:397-431): look the tensor up, check its rank and
// repack it -- per expert for a 3-D tensor, slabs back to back.
int rein_gguf_load_for_matvec(const rein_gguf* g, const char* name, uint8_t* dst, size_t dst_len, int* out_fmt,
                              rein_gguf_dims* dims)
{
    rein_gguf_tensor t;
    if (int rc = rein_gguf_tensor_by_name(g, name, &t)) return rc;
    if (t.n_dims != 2 && t.n_dims != 3)
        return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": expected 2D or 3D, got " + std::to_string(t.n_dims) + "D");
    // a 3-D tensor is a stack of experts and takes the expert formats, a 2-D one the dense formats
    const int label = t.n_dims == 3 ? rein_ingest_expert_format(t.ggml_type) : rein_ingest_format(t.ggml_type);
    if (!label)
        return fail(REIN_E_BAD_FORMAT, std::string("tensor ") + name + ": no " + (t.n_dims == 3 ? "MoE " : "") +
                                           "kernels for ggml type " + std::to_string(t.ggml_type) +
                                           (t.n_dims == 3 ? " (experts must be Q4_K, Q5_K, Q6_K, Q8_0 or Q5_1)" : ""));
    if (t.dims[0] > 0xFFFFFFFFull || t.dims[1] > 0xFFFFFFFFull || t.dims[2] > 0xFFFFFFFFull)
        return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": dimension above 32 bits");
    const size_t in_dim = (size_t)t.dims[0], out_dim = (size_t)t.dims[1], n_expert = (size_t)t.dims[2];
    if (!in_dim || !out_dim || !n_expert) return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": empty dimension");
    uint64_t src_block, src_block_bytes;
    ggml_geometry((uint32_t)t.ggml_type, &src_block, &src_block_bytes);
    const size_t mult = src_block > 32 ? (size_t)src_block : 32;      // rows are whole blocks; BF16 rows become Q8_0 blocks
    if (in_dim % mult)
        return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": in_dim " + std::to_string(in_dim) + " is not a multiple of " +
                                          std::to_string(mult));
    const size_t per = rein_repacked_len(label, in_dim, out_dim);
    const size_t src_per = (size_t)(t.byte_size / n_expert);
    if (n_expert > 1 && per % 16)
        return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": expert slabs of " + std::to_string(per) +
                                          " bytes are not 16-byte multiples (out_dim must be a multiple of 8)");
    if (dims) { dims->in_dim = (unsigned)in_dim; dims->out_dim = (unsigned)out_dim; dims->n_expert = (unsigned)n_expert; dims->bytes_per_expert = per; }
    if (out_fmt) *out_fmt = label;
    if (!dst) return REIN_OK;                              // size query
    if (dst_len < per * n_expert)
        return fail(REIN_E_BAD_SHAPE, std::string("tensor ") + name + ": destination holds " + std::to_string(dst_len) + " bytes, " +
                                          std::to_string(per * n_expert) + " needed");
    for (size_t e = 0; e < n_expert; e++) {
        const int rc = t.n_dims == 3 ? rein_repack_for_matvec(label, t.data + e * src_per, in_dim, out_dim, dst + e * per)
                                     : rein_ingest_for_matvec(t.ggml_type, t.data + e * src_per, in_dim, out_dim, dst + e * per, nullptr);
        if (rc) return rc;
    }
    return REIN_OK;
}

}  // extern "C"
