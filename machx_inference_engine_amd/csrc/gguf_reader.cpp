// gguf_reader.cpp — memory-mapped GGUF (v2 / v3) reader: the on-disk step on the input side of the
// quantized-matmul path.  Mirrors the reference's GgufReader (include/ie/gguf.hpp:72-117,
// src/loaders/gguf_reader.cpp): header, key/value metadata, tensor directory, data blob aligned to
// general.alignment, and split models ("...-00001-of-0000N.gguf": metadata in the first shard,
// tensors from every shard).  Tensor data is never copied: every entry points into the mapping, in
// the GGUF block layouts the kernels read directly.
//
// Container:  "GGUF" u32 | version u32 | n_tensors u64 | n_kv u64 | n_kv x {key str, type u32, value}
//             | n_tensors x {name str, n_dims u32, dims u64[n_dims], ggml_type u32, offset u64}
//             | pad to alignment | data.     str = u64 length + bytes (no terminator).
#include <errno.h>
#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <vector>

#include "../../include/mxq.h"

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

struct Mapping {
    int fd = -1;
    const uint8_t* base = nullptr;
    size_t size = 0;
};

struct Gguf {
    std::vector<Mapping> maps;
    uint32_t version = 0;
    uint64_t alignment = 32;
    uint64_t data_off = 0;   // of the first shard
    std::vector<mx_gguf_kv_t> kvs;
    std::vector<mx_gguf_tensor_t> tensors;
};

// bytes per block / elements per block of a ggml type id; {0, 0} = not a type this reader sizes
void type_size(uint32_t t, uint32_t* bytes, uint32_t* elems) {
    static const struct { uint32_t id, bytes, elems; } kTypes[] = {
        {0, 4, 1},      {1, 2, 1},      {2, 18, 32},    {3, 20, 32},    {6, 22, 32},    {7, 24, 32},   {8, 34, 32},   {9, 36, 32},
        {10, 84, 256},  {11, 110, 256}, {12, 144, 256}, {13, 176, 256}, {14, 210, 256}, {15, 292, 256}, {24, 1, 1},   {25, 2, 1},
        {26, 4, 1},     {27, 8, 1},     {28, 8, 1},     {30, 2, 1},     {39, 17, 32},
    };
    *bytes = *elems = 0;
    for (const auto& e : kTypes)
        if (e.id == t) {
            *bytes = e.bytes;
            *elems = e.elems;
        }
}

// size of one scalar of a metadata value type; 0 for string / array / unknown
size_t scalar_size(uint32_t t) {
    switch (t) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
    }
    return 0;
}

struct Cursor {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    bool need(size_t n) {
        if (!ok || (size_t)(end - p) < n) ok = false;
        return ok;
    }
    uint32_t u32() {
        uint32_t v = 0;
        if (need(4)) { memcpy(&v, p, 4); p += 4; }
        return v;
    }
    uint64_t u64() {
        uint64_t v = 0;
        if (need(8)) { memcpy(&v, p, 8); p += 8; }
        return v;
    }
    // string: returns pointer + length, advances
    const char* str(uint64_t* len) {
        *len = u64();
        if (!need(*len)) { *len = 0; return nullptr; }
        const char* s = reinterpret_cast<const char*>(p);
        p += *len;
        return s;
    }
    void skip_value(uint32_t type, int depth = 0) {
        if (!ok) return;
        if (const size_t sz = scalar_size(type)) { if (need(sz)) p += sz; return; }
        if (type == 8) { uint64_t n; str(&n); return; }
        if (type == 9 && depth == 0) {
            const uint32_t inner = u32();
            const uint64_t n = u64();
            if (const size_t sz = scalar_size(inner)) {
                if (n > (uint64_t)(end - p) / sz) { ok = false; return; }
                p += n * sz;
            } else if (inner == 8) {
                for (uint64_t i = 0; i < n && ok; ++i) { uint64_t l; str(&l); }
            } else {
                ok = false;   // nested arrays are not produced by any writer this engine reads
            }
            return;
        }
        ok = false;
    }
};

bool key_is(const mx_gguf_kv_t& kv, const char* s) { return kv.key_len == strlen(s) && memcmp(kv.key, s, kv.key_len) == 0; }

uint64_t kv_uint(const mx_gguf_kv_t& kv) {
    uint64_t v = 0;
    const size_t sz = scalar_size(kv.type);
    if (sz && kv.type != 6 && kv.type != 12) memcpy(&v, kv.payload, sz);
    return v;
}

int map_file(const std::string& path, Mapping* m) {
    m->fd = ::open(path.c_str(), O_RDONLY);
    if (m->fd < 0) return fail(MX_ERR_IO, "open(" + path + ") failed: " + strerror(errno));
    struct stat st;
    if (fstat(m->fd, &st) != 0 || st.st_size < 24) {
        ::close(m->fd);
        return fail(MX_ERR_FORMAT, path + ": not a GGUF file (shorter than its header)");
    }
    m->size = (size_t)st.st_size;
    void* p = mmap(nullptr, m->size, PROT_READ, MAP_PRIVATE, m->fd, 0);
    if (p == MAP_FAILED) {
        ::close(m->fd);
        return fail(MX_ERR_IO, "mmap(" + path + ") failed: " + strerror(errno));
    }
    m->base = static_cast<const uint8_t*>(p);
    return MX_OK;
}

// Parses one shard; metadata is kept from the primary shard only, tensors from every shard.
int parse_shard(Gguf* g, const Mapping& m, bool primary, const std::string& path) {
    Cursor c{m.base, m.base + m.size};
    if (c.u32() != 0x46554747u) return fail(MX_ERR_FORMAT, path + ": bad magic");
    const uint32_t version = c.u32();
    if (version < 2 || version > 3) return fail(MX_ERR_FORMAT, path + ": GGUF version " + std::to_string(version) + " not supported (2 or 3)");
    const uint64_t n_tensors = c.u64(), n_kv = c.u64();
    if (n_kv > m.size || n_tensors > m.size) return fail(MX_ERR_FORMAT, path + ": counts exceed the file size");
    uint64_t alignment = 32;
    for (uint64_t i = 0; i < n_kv; ++i) {
        mx_gguf_kv_t kv{};
        kv.key = c.str(&kv.key_len);
        kv.type = c.u32();
        if (kv.type == 9) {
            Cursor peek = c;
            kv.inner_type = peek.u32();
            kv.n_array = peek.u64();
            kv.payload = peek.p;
        } else if (kv.type == 8) {
            kv.payload = c.p;   // u64 length + bytes
        } else {
            kv.payload = c.p;
        }
        c.skip_value(kv.type);
        if (!c.ok) return fail(MX_ERR_FORMAT, path + ": truncated or malformed metadata at key " + std::to_string(i));
        if (key_is(kv, "general.alignment")) alignment = kv_uint(kv);
        if (primary) g->kvs.push_back(kv);
    }
    if (alignment == 0 || (alignment & (alignment - 1))) return fail(MX_ERR_FORMAT, path + ": general.alignment is not a power of two");
    const size_t first = g->tensors.size();
    for (uint64_t i = 0; i < n_tensors; ++i) {
        mx_gguf_tensor_t t{};
        t.name = c.str(&t.name_len);
        t.n_dims = c.u32();
        if (t.n_dims > 4) return fail(MX_ERR_FORMAT, path + ": tensor " + std::to_string(i) + " has more than 4 dimensions");
        uint64_t n_elem = 1;
        for (uint32_t d = 0; d < 4; ++d) t.shape[d] = 1;
        for (uint32_t d = 0; d < t.n_dims; ++d) {
            t.shape[d] = c.u64();
            if (t.shape[d] != 0 && n_elem > UINT64_MAX / t.shape[d]) return fail(MX_ERR_FORMAT, path + ": tensor shape overflows");
            n_elem *= t.shape[d];
        }
        t.ggml_type = c.u32();
        t.offset_in_data = c.u64();
        if (!c.ok) return fail(MX_ERR_FORMAT, path + ": truncated tensor directory at entry " + std::to_string(i));
        uint32_t bytes, elems;
        type_size(t.ggml_type, &bytes, &elems);
        if (bytes) {
            if (t.shape[0] % elems) return fail(MX_ERR_FORMAT, path + ": tensor row length is not a whole number of blocks");
            // no format here packs more than 8 elements into a byte: anything larger cannot lie in this file
            // (and would overflow the size computation)
            if (n_elem / 8 > m.size) return fail(MX_ERR_FORMAT, path + ": tensor " + std::to_string(i) + " is larger than the file");
            t.nbytes = n_elem / elems * bytes;
        }
        g->tensors.push_back(t);
    }
    const uint64_t dir_end = (uint64_t)(c.p - m.base);
    const uint64_t data_off = (dir_end + alignment - 1) / alignment * alignment;
    for (size_t i = first; i < g->tensors.size(); ++i) {
        mx_gguf_tensor_t& t = g->tensors[i];
        if (data_off > m.size || t.offset_in_data > m.size - data_off || t.nbytes > m.size - data_off - t.offset_in_data)
            return fail(MX_ERR_FORMAT, path + ": tensor '" + std::string(t.name, t.name_len) + "' lies outside the file");
        t.data = m.base + data_off + t.offset_in_data;
    }
    if (primary) {
        g->version = version;
        g->alignment = alignment;
        g->data_off = data_off;
    }
    return MX_OK;
}

// "<prefix>-NNNNN-of-MMMMM.gguf" -> prefix, shard number, shard count
bool parse_split_name(const std::string& path, std::string* prefix, unsigned* no, unsigned* count) {
    const size_t n = path.size();
    if (n < 20 || path.compare(n - 5, 5, ".gguf") != 0) return false;
    const std::string tail = path.substr(n - 20, 15);   // -NNNNN-of-MMMMM
    if (tail[0] != '-' || tail.compare(6, 4, "-of-") != 0) return false;
    for (int i : {1, 2, 3, 4, 5, 10, 11, 12, 13, 14})
        if (tail[i] < '0' || tail[i] > '9') return false;
    *no = (unsigned)atoi(tail.substr(1, 5).c_str());
    *count = (unsigned)atoi(tail.substr(10, 5).c_str());
    *prefix = path.substr(0, n - 20);
    return true;
}

void destroy(Gguf* g) {
    for (const Mapping& m : g->maps) {
        if (m.base) munmap(const_cast<uint8_t*>(m.base), m.size);
        if (m.fd >= 0) ::close(m.fd);
    }
    delete g;
}

}  // namespace

extern "C" {

const char* mx_gguf_last_error(void) { return g_err.c_str(); }

int mx_gguf_open(const char* path, void** handle) {
    if (!path || !handle) return MX_ERR_NULL;
    *handle = nullptr;
    Gguf* g = new Gguf();
    Mapping m;
    if (int rc = map_file(path, &m)) { delete g; return rc; }
    g->maps.push_back(m);
    if (int rc = parse_shard(g, m, true, path)) { destroy(g); return rc; }
    uint64_t split_count = 0;
    for (const auto& kv : g->kvs)
        if (key_is(kv, "split.count")) split_count = kv_uint(kv);
    if (split_count > 1) {
        std::string prefix;
        unsigned no = 0, count = 0;
        if (!parse_split_name(path, &prefix, &no, &count) || count != split_count) {
            destroy(g);
            return fail(MX_ERR_FORMAT, std::string(path) + ": split.count > 1 but the name is not '...-NNNNN-of-MMMMM.gguf' with that count");
        }
        if (no != 1) { destroy(g); return fail(MX_ERR_FORMAT, "open the first shard (-00001-of-...) of a split GGUF"); }
        for (unsigned s = 2; s <= count; ++s) {
            char tail[32];
            snprintf(tail, sizeof tail, "-%05u-of-%05u.gguf", s, count);
            const std::string sp = prefix + tail;
            Mapping sm;
            if (int rc = map_file(sp, &sm)) { destroy(g); return rc; }
            g->maps.push_back(sm);
            if (int rc = parse_shard(g, sm, false, sp)) { destroy(g); return rc; }
        }
        for (const auto& kv : g->kvs)
            if (key_is(kv, "split.tensors.count") && kv_uint(kv) != g->tensors.size()) {
                destroy(g);
                return fail(MX_ERR_FORMAT, "split.tensors.count does not match the tensors found in the shards");
            }
    }
    *handle = g;
    return MX_OK;
}

int mx_gguf_close(void* handle) {
    if (!handle) return MX_ERR_NULL;
    destroy(static_cast<Gguf*>(handle));
    return MX_OK;
}

int mx_gguf_info(const void* handle, uint32_t* version, uint64_t* n_tensors, uint64_t* n_kv, uint64_t* alignment, uint64_t* tensor_data_offset) {
    if (!handle) return MX_ERR_NULL;
    const Gguf* g = static_cast<const Gguf*>(handle);
    if (version) *version = g->version;
    if (n_tensors) *n_tensors = g->tensors.size();
    if (n_kv) *n_kv = g->kvs.size();
    if (alignment) *alignment = g->alignment;
    if (tensor_data_offset) *tensor_data_offset = g->data_off;
    return MX_OK;
}

int mx_gguf_tensor(const void* handle, uint64_t i, mx_gguf_tensor_t* out) {
    if (!handle || !out) return MX_ERR_NULL;
    const Gguf* g = static_cast<const Gguf*>(handle);
    if (i >= g->tensors.size()) return MX_ERR_SHAPE;
    *out = g->tensors[i];
    return MX_OK;
}

int mx_gguf_find_tensor(const void* handle, const char* name, uint64_t* index) {
    if (!handle || !name || !index) return MX_ERR_NULL;
    const Gguf* g = static_cast<const Gguf*>(handle);
    const size_t n = strlen(name);
    for (size_t i = 0; i < g->tensors.size(); ++i)
        if (g->tensors[i].name_len == n && memcmp(g->tensors[i].name, name, n) == 0) {
            *index = i;
            return MX_OK;
        }
    return MX_ERR_NOT_FOUND;
}

int mx_gguf_kv(const void* handle, uint64_t i, mx_gguf_kv_t* out) {
    if (!handle || !out) return MX_ERR_NULL;
    const Gguf* g = static_cast<const Gguf*>(handle);
    if (i >= g->kvs.size()) return MX_ERR_SHAPE;
    *out = g->kvs[i];
    return MX_OK;
}

int mx_gguf_find_kv(const void* handle, const char* key, uint64_t* index) {
    if (!handle || !key || !index) return MX_ERR_NULL;
    const Gguf* g = static_cast<const Gguf*>(handle);
    for (size_t i = 0; i < g->kvs.size(); ++i)
        if (key_is(g->kvs[i], key)) {
            *index = i;
            return MX_OK;
        }
    return MX_ERR_NOT_FOUND;
}

}  // extern "C"
