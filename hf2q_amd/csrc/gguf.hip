// GGUF v3 reader: header, metadata and tensor directory of a memory-mapped file, and upload of a
// tensor's raw GGML blocks to the device.  The byte format is the one hf2q's own writer emits
// (src/backends/gguf/types.rs:20-32, 96-188; src/backends/gguf/writer.rs:171-258): little endian,
//   "GGUF" | u32 version | u64 tensor_count | u64 kv_count
//   kv:     string key | u32 type | payload         (string = u64 length | bytes,
//                                                    array  = u32 elem type | u64 count | elements)
//   tensor: string name | u32 n_dims | u64 dims[n_dims] (innermost first) | u32 ggml type | u64 offset
//   padding to the alignment (32, or the metadata key general.alignment), then the tensor data;
//   offsets are relative to the start of the data section.
// Host code only; nothing here launches a kernel.
#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "hq_internal.h"

namespace hq {
namespace {

// ggml_type.rs:18-53, 60-135: elements and bytes per block of every type id hf2q knows.
struct TypeGeom {
    uint32_t id, block_elems, block_bytes;
};
constexpr TypeGeom kTypes[] = {
    {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},    {7, 32, 24},   {8, 32, 34},
    {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292},
    {16, 256, 66},  {17, 256, 74},  {18, 256, 98},  {19, 256, 50},  {20, 32, 18},   {21, 256, 110}, {22, 256, 82},
    {23, 256, 136}, {29, 256, 56},  {30, 1, 2},     {34, 256, 54},  {35, 256, 66},  {39, 32, 17},
};
const TypeGeom* geom_of(uint32_t id) {
    for (const TypeGeom& g : kTypes)
        if (g.id == id) return &g;
    return nullptr;
}

enum : uint32_t { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 };  // types.rs:41-53
constexpr uint32_t kScalarBytes[] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};

struct MetaEntry {
    uint32_t type;        // value type; for arrays the element type is in elem_type
    uint32_t elem_type;
    uint64_t count;       // arrays: elements
    const uint8_t* data;  // scalars: the value; strings: the bytes (count = length); arrays: the first element
};

}  // namespace
}  // namespace hq

using namespace hq;

struct hq_gguf {
    int fd = -1;
    const uint8_t* base = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    uint64_t alignment = 32;
    uint64_t data_start = 0;
    std::vector<std::string> names;
    std::vector<hq_gguf_tensor_info> infos;
    std::unordered_map<std::string, size_t> by_name;
    std::vector<std::string> keys;
    std::unordered_map<std::string, MetaEntry> meta;
};

namespace {

// Bounds-checked cursor over the mapping.
struct Cursor {
    const uint8_t* base;
    size_t size, pos;
    bool ok = true;
    const uint8_t* take(size_t n) {
        if (!ok || n > size - pos) {
            ok = false;
            return nullptr;
        }
        const uint8_t* p = base + pos;
        pos += n;
        return p;
    }
    template <typename T>
    T get() {
        T v{};
        if (const uint8_t* p = take(sizeof(T))) memcpy(&v, p, sizeof(T));
        return v;
    }
    // string = u64 length | bytes (types.rs:96-101)
    bool str(const uint8_t** p, uint64_t* len) {
        *len = get<uint64_t>();
        if (!ok || *len > size - pos) return ok = false;
        *p = take((size_t)*len);
        return ok;
    }
};

void destroy(hq_gguf* g) {
    if (!g) return;
    if (g->base) munmap(const_cast<uint8_t*>(g->base), g->size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

int parse(hq_gguf* g, const char* path) {
    Cursor c{g->base, g->size, 0};
    const uint8_t* magic = c.take(4);
    if (!magic || memcmp(magic, "GGUF", 4) != 0) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s is not a GGUF file", path);
    g->version = c.get<uint32_t>();
    if (g->version != 3 && g->version != 2)
        return fail(HQ_ERR_UNSUPPORTED, "hq_gguf_open: %s: GGUF version %u (2 or 3 expected)", path, g->version);
    const uint64_t n_tensors = c.get<uint64_t>(), n_kv = c.get<uint64_t>();
    if (!c.ok || n_tensors > g->size / 24 || n_kv > g->size / 12)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: truncated or corrupt header", path);

    for (uint64_t i = 0; i < n_kv; ++i) {  // types.rs:103-188
        const uint8_t* kp;
        uint64_t klen;
        if (!c.str(&kp, &klen)) break;
        MetaEntry e{};
        e.type = c.get<uint32_t>();
        if (!c.ok || e.type > T_F64) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: metadata value type %u", path, e.type);
        if (e.type == T_STR) {
            if (!c.str(&e.data, &e.count)) break;
        } else if (e.type == T_ARR) {
            e.elem_type = c.get<uint32_t>();
            e.count = c.get<uint64_t>();
            if (!c.ok || e.elem_type > T_F64 || e.elem_type == T_ARR)
                return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: array element type %u", path, e.elem_type);
            e.data = g->base + c.pos;
            if (e.elem_type == T_STR) {
                for (uint64_t j = 0; j < e.count && c.ok; ++j) {
                    const uint8_t* sp;
                    uint64_t sl;
                    c.str(&sp, &sl);
                }
            } else {
                if (e.count > (g->size - c.pos) / kScalarBytes[e.elem_type]) c.ok = false;
                else c.take((size_t)e.count * kScalarBytes[e.elem_type]);
            }
        } else {
            e.count = 1;
            e.data = c.take(kScalarBytes[e.type]);
        }
        if (!c.ok) break;
        std::string key(reinterpret_cast<const char*>(kp), (size_t)klen);
        g->keys.push_back(key);
        g->meta.emplace(std::move(key), e);
    }
    if (!c.ok) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: truncated metadata", path);
    auto al = g->meta.find("general.alignment");
    if (al != g->meta.end() && al->second.type == T_U32) {
        uint32_t v;
        memcpy(&v, al->second.data, 4);
        if (v == 0 || (v & (v - 1))) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: general.alignment %u", path, v);
        g->alignment = v;
    }

    for (uint64_t i = 0; i < n_tensors; ++i) {  // writer.rs:186-222
        const uint8_t* np;
        uint64_t nlen;
        if (!c.str(&np, &nlen)) break;
        hq_gguf_tensor_info ti{};
        ti.n_dims = c.get<uint32_t>();
        if (!c.ok || ti.n_dims > 4) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: tensor with %u dimensions", path, ti.n_dims);
        uint64_t elems = 1;
        for (uint32_t d = 0; d < 4; ++d) ti.dims[d] = 1;
        for (uint32_t d = 0; d < ti.n_dims; ++d) {
            ti.dims[d] = c.get<uint64_t>();
            if (ti.dims[d] != 0 && elems > UINT64_MAX / ti.dims[d]) c.ok = false;
            elems *= ti.dims[d];
        }
        ti.ggml_type = c.get<uint32_t>();
        ti.data_offset = c.get<uint64_t>();  // relative for now
        if (!c.ok) break;
        const TypeGeom* tg = geom_of(ti.ggml_type);
        std::string name(reinterpret_cast<const char*>(np), (size_t)nlen);
        if (!tg) return fail(HQ_ERR_UNSUPPORTED, "hq_gguf_open: %s: tensor %s has unknown ggml type %u", path, name.c_str(), ti.ggml_type);
        // rows are contiguous and whole blocks (quantizer.rs:57-71)
        if (ti.n_dims && ti.dims[0] % tg->block_elems)
            return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: tensor %s: row length %llu is not a multiple of the block size %u",
                        path, name.c_str(), (unsigned long long)ti.dims[0], tg->block_elems);
        if (elems / tg->block_elems > UINT64_MAX / tg->block_bytes)
            return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: tensor %s: %llu elements do not fit a 64-bit byte count", path,
                        name.c_str(), (unsigned long long)elems);
        ti.byte_len = elems / tg->block_elems * tg->block_bytes;
        g->by_name.emplace(name, g->infos.size());
        g->names.push_back(std::move(name));
        g->infos.push_back(ti);
    }
    if (!c.ok) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: truncated tensor directory", path);
    g->data_start = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    for (size_t i = 0; i < g->infos.size(); ++i) {
        hq_gguf_tensor_info& ti = g->infos[i];
        if (ti.data_offset % g->alignment)
            return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: tensor %s: offset %llu breaks the %llu-byte alignment", path,
                        g->names[i].c_str(), (unsigned long long)ti.data_offset, (unsigned long long)g->alignment);
        if (g->data_start > g->size || ti.data_offset > g->size - g->data_start || ti.byte_len > g->size - g->data_start - ti.data_offset)
            return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: %s: tensor %s reaches past the end of the file", path, g->names[i].c_str());
        ti.data_offset += g->data_start;  // absolute from here on
    }
    return HQ_OK;
}

const MetaEntry* find_meta(const hq_gguf* g, const char* key, const char* fn) {
    if (!g || !key) {
        fail(HQ_ERR_INVALID_ARGUMENT, "%s: null argument", fn);
        return nullptr;
    }
    auto it = g->meta.find(key);
    if (it == g->meta.end()) {
        fail(HQ_ERR_INVALID_ARGUMENT, "%s: no metadata key %s", fn, key);
        return nullptr;
    }
    return &it->second;
}

}  // namespace

extern "C" {

int hq_gguf_open(const char* path, hq_gguf** out) {
    if (!path || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: null argument");
    *out = nullptr;
    hq_gguf* g = new hq_gguf;
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (g->fd < 0 || fstat(g->fd, &st) != 0) {
        const int rc = fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: cannot open %s: %s", path, strerror(errno));
        destroy(g);
        return rc;
    }
    g->size = (size_t)st.st_size;
    void* m = g->size ? mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0) : MAP_FAILED;
    if (m == MAP_FAILED) {
        const int rc = fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_open: cannot map %s (%zu bytes)", path, g->size);
        destroy(g);
        return rc;
    }
    g->base = static_cast<const uint8_t*>(m);
    if (int rc = parse(g, path)) {
        destroy(g);
        return rc;
    }
    *out = g;
    return HQ_OK;
}

void hq_gguf_close(hq_gguf* g) { destroy(g); }

uint64_t hq_gguf_tensor_count(const hq_gguf* g) { return g ? g->infos.size() : 0; }
uint64_t hq_gguf_metadata_count(const hq_gguf* g) { return g ? g->keys.size() : 0; }
uint64_t hq_gguf_alignment(const hq_gguf* g) { return g ? g->alignment : 0; }

const char* hq_gguf_tensor_name(const hq_gguf* g, uint64_t index) {
    return g && index < g->names.size() ? g->names[(size_t)index].c_str() : nullptr;
}

const char* hq_gguf_metadata_key(const hq_gguf* g, uint64_t index) {
    return g && index < g->keys.size() ? g->keys[(size_t)index].c_str() : nullptr;
}

int hq_gguf_tensor_info_by_name(const hq_gguf* g, const char* name, hq_gguf_tensor_info* out) {
    if (!g || !name || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_tensor_info_by_name: null argument");
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_tensor_info_by_name: no tensor %s", name);
    *out = g->infos[it->second];
    return HQ_OK;
}

int hq_gguf_metadata_u64(const hq_gguf* g, const char* key, uint64_t* out) {
    const MetaEntry* e = find_meta(g, key, "hq_gguf_metadata_u64");
    if (!e || !out) return e ? fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_u64: null out") : HQ_ERR_INVALID_ARGUMENT;
    uint64_t v = 0;
    switch (e->type) {
        case T_U8: case T_BOOL: v = *e->data; break;
        case T_U16: { uint16_t t; memcpy(&t, e->data, 2); v = t; break; }
        case T_U32: { uint32_t t; memcpy(&t, e->data, 4); v = t; break; }
        case T_U64: memcpy(&v, e->data, 8); break;
        case T_I8: case T_I16: case T_I32: case T_I64: {
            int64_t s = 0;
            if (e->type == T_I8) s = (int8_t)*e->data;
            else if (e->type == T_I16) { int16_t t; memcpy(&t, e->data, 2); s = t; }
            else if (e->type == T_I32) { int32_t t; memcpy(&t, e->data, 4); s = t; }
            else memcpy(&s, e->data, 8);
            if (s < 0) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_u64: %s is negative", key);
            v = (uint64_t)s;
            break;
        }
        default: return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_u64: %s is not an integer (type %u)", key, e->type);
    }
    *out = v;
    return HQ_OK;
}

int hq_gguf_metadata_f64(const hq_gguf* g, const char* key, double* out) {
    const MetaEntry* e = find_meta(g, key, "hq_gguf_metadata_f64");
    if (!e || !out) return e ? fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_f64: null out") : HQ_ERR_INVALID_ARGUMENT;
    if (e->type == T_F32) { float t; memcpy(&t, e->data, 4); *out = t; return HQ_OK; }
    if (e->type == T_F64) { memcpy(out, e->data, 8); return HQ_OK; }
    return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_f64: %s is not a float (type %u)", key, e->type);
}

int hq_gguf_metadata_string(const hq_gguf* g, const char* key, const char** out, uint64_t* len) {
    const MetaEntry* e = find_meta(g, key, "hq_gguf_metadata_string");
    if (!e || !out || !len) return e ? fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_string: null out") : HQ_ERR_INVALID_ARGUMENT;
    if (e->type != T_STR) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_metadata_string: %s is not a string (type %u)", key, e->type);
    *out = reinterpret_cast<const char*>(e->data);  // not NUL-terminated
    *len = e->count;
    return HQ_OK;
}

const void* hq_gguf_tensor_data(const hq_gguf* g, const char* name, uint64_t* byte_len) {
    hq_gguf_tensor_info ti;
    if (hq_gguf_tensor_info_by_name(g, name, &ti)) return nullptr;
    if (byte_len) *byte_len = ti.byte_len;
    return g->base + ti.data_offset;
}

int hq_gguf_load_tensor(const hq_gguf* g, const char* name, void* stream, void* dev_dst, size_t dst_bytes) {
    hq_gguf_tensor_info ti;
    if (int rc = hq_gguf_tensor_info_by_name(g, name, &ti)) return rc;
    if (ti.byte_len == 0) return HQ_OK;
    if (!dev_dst || dst_bytes < ti.byte_len)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gguf_load_tensor: %s needs %llu bytes, destination has %zu", name,
                    (unsigned long long)ti.byte_len, dev_dst ? dst_bytes : (size_t)0);
    // Load-time path: the source is a pageable file mapping, so the call waits for the copy; the file
    // may be closed right after it returns.
    if (int rc = check_hip(hipMemcpyAsync(dev_dst, g->base + ti.data_offset, (size_t)ti.byte_len, hipMemcpyHostToDevice,
                                          (hipStream_t)stream),
                           "hipMemcpyAsync(gguf tensor)"))
        return rc;
    return check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize(gguf tensor)");
}

}  // extern "C"
