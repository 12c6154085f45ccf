// GGUF tensor directory reader and the prepared-weights container (weights_io.h).
#include "llaminar_amd/weights_io.h"

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

#include "llaminar_amd/ql_api.h"
#include "llaminar_amd/ql_blocks.h"

namespace
{
    thread_local char g_error[512] = "";

    bool fail(const char *fmt, ...)
    {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(g_error, sizeof g_error, fmt, ap);
        va_end(ap);
        return false;
    }

    // ---- GGUF ---------------------------------------------------------------------------
    constexpr uint32_t GGUF_MAGIC = 0x46554747u; // "GGUF"
    enum : uint32_t
    {
        GV_U8 = 0, GV_I8, GV_U16, GV_I16, GV_U32, GV_I32, GV_F32, GV_BOOL, GV_STRING, GV_ARRAY, GV_U64, GV_I64, GV_F64,
        GV_COUNT
    };
    // bytes of a scalar metadata value; 0 for strings and arrays
    constexpr uint32_t GV_BYTES[GV_COUNT] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};

    struct TypeSize
    {
        uint32_t block_bytes, block_elems;
    };
    // ggml tensor type id -> block geometry (0 = unknown here)
    TypeSize type_size(uint32_t t)
    {
        switch (t)
        {
        case 0: return {4, 1};      // F32
        case 1: return {2, 1};      // F16
        case 2: return {18, 32};    // Q4_0
        case 3: return {20, 32};    // Q4_1
        case 6: return {22, 32};    // Q5_0
        case 7: return {24, 32};    // Q5_1
        case 8: return {34, 32};    // Q8_0
        case 9: return {36, 32};    // Q8_1
        case 10: return {84, 256};  // Q2_K
        case 11: return {110, 256}; // Q3_K
        case 12: return {144, 256}; // Q4_K
        case 13: return {176, 256}; // Q5_K
        case 14: return {210, 256}; // Q6_K
        case 15: return {292, 256}; // Q8_K
        case 16: return {66, 256};  // IQ2_XXS
        case 17: return {74, 256};  // IQ2_XS
        case 18: return {98, 256};  // IQ3_XXS
        case 19: return {50, 256};  // IQ1_S
        case 20: return {18, 32};   // IQ4_NL
        case 21: return {110, 256}; // IQ3_S
        case 22: return {82, 256};  // IQ2_S
        case 23: return {136, 256}; // IQ4_XS
        case 24: return {1, 1};     // I8
        case 25: return {2, 1};     // I16
        case 26: return {4, 1};     // I32
        case 27: return {8, 1};     // I64
        case 28: return {8, 1};     // F64
        case 29: return {56, 256};  // IQ1_M
        case 30: return {2, 1};     // BF16
        default: return {0, 0};
        }
    }
    uint8_t type_fmt(uint32_t t)
    {
        switch (t)
        {
        case 12: return LLAM_FMT_Q4_K;
        case 14: return LLAM_FMT_Q6_K;
        case 21: return LLAM_FMT_IQ3_S;
        default: return 0;
        }
    }

    struct MetaValue
    {
        uint32_t type;
        uint64_t bits;   // scalar payload, zero-extended
        std::string str; // GV_STRING
    };

    struct Tensor
    {
        std::string name;
        uint32_t type, n_dims;
        uint64_t dims[4], offset, nbytes;
    };

    struct Gguf
    {
        const uint8_t *base = nullptr;
        uint64_t size = 0;
        uint64_t data_start = 0;
        uint32_t version = 0;
        std::vector<Tensor> tensors;
        std::unordered_map<std::string, size_t> by_name;
        std::unordered_map<std::string, MetaValue> meta;
        ~Gguf()
        {
            if (base)
                munmap(const_cast<uint8_t *>(base), size);
        }
    };

    // bounds-checked cursor over the mapping
    struct Cursor
    {
        const uint8_t *base;
        uint64_t size, at;
        bool take(void *dst, uint64_t n)
        {
            if (n > size - at)
                return false;
            memcpy(dst, base + at, n);
            at += n;
            return true;
        }
        bool skip(uint64_t n)
        {
            if (n > size - at)
                return false;
            at += n;
            return true;
        }
        template <class T>
        bool get(T &v)
        {
            return take(&v, sizeof v);
        }
        bool string(std::string &s, uint64_t max_len)
        {
            uint64_t n;
            if (!get(n) || n > max_len || n > size - at)
                return false;
            s.assign(reinterpret_cast<const char *>(base + at), (size_t)n);
            at += n;
            return true;
        }
    };

    bool skip_value(Cursor &c, uint32_t type, int depth)
    {
        if (type >= GV_COUNT)
            return false;
        if (type == GV_STRING)
        {
            uint64_t n;
            return c.get(n) && c.skip(n);
        }
        if (type == GV_ARRAY)
        {
            uint32_t et;
            uint64_t n;
            if (depth > 4 || !c.get(et) || !c.get(n) || et >= GV_COUNT)
                return false;
            if (GV_BYTES[et])
                return n <= (c.size - c.at) / GV_BYTES[et] && c.skip(n * GV_BYTES[et]);
            for (uint64_t i = 0; i < n; ++i)
                if (!skip_value(c, et, depth + 1))
                    return false;
            return true;
        }
        return c.skip(GV_BYTES[type]);
    }

    bool parse(Gguf &g)
    {
        Cursor c{g.base, g.size, 0};
        uint32_t magic;
        uint64_t n_tensors, n_kv;
        if (!c.get(magic) || magic != GGUF_MAGIC)
            return fail("not a GGUF file (magic)");
        if (!c.get(g.version) || (g.version != 2 && g.version != 3))
            return fail("GGUF version %u: only 2 and 3 are read", g.version);
        if (!c.get(n_tensors) || !c.get(n_kv))
            return fail("truncated header");
        // every tensor entry takes at least 8 + 4 + 4 + 8 bytes, every pair at least 8 + 4
        if (n_tensors > g.size / 24 || n_kv > g.size / 12)
            return fail("header counts (%llu tensors, %llu metadata pairs) exceed the file",
                        (unsigned long long)n_tensors, (unsigned long long)n_kv);
        for (uint64_t i = 0; i < n_kv; ++i)
        {
            std::string key;
            uint32_t type;
            if (!c.string(key, 65535) || !c.get(type) || type >= GV_COUNT)
                return fail("metadata pair %llu is malformed", (unsigned long long)i);
            MetaValue v{type, 0, {}};
            if (type == GV_STRING)
            {
                if (!c.string(v.str, g.size))
                    return fail("metadata string '%s' runs past the end of the file", key.c_str());
            }
            else if (type == GV_ARRAY)
            {
                if (!skip_value(c, type, 0))
                    return fail("metadata array '%s' is malformed", key.c_str());
                continue; // arrays (vocabularies, merges) are not kept
            }
            else if (!c.take(&v.bits, GV_BYTES[type]))
                return fail("metadata value '%s' runs past the end of the file", key.c_str());
            g.meta.emplace(std::move(key), std::move(v));
        }
        g.tensors.reserve((size_t)n_tensors);
        for (uint64_t i = 0; i < n_tensors; ++i)
        {
            Tensor t{};
            if (!c.string(t.name, 65535) || !c.get(t.n_dims) || t.n_dims < 1 || t.n_dims > 4)
                return fail("tensor entry %llu is malformed", (unsigned long long)i);
            t.dims[0] = t.dims[1] = t.dims[2] = t.dims[3] = 1;
            for (uint32_t d = 0; d < t.n_dims; ++d)
                if (!c.get(t.dims[d]) || t.dims[d] == 0)
                    return fail("tensor '%s': bad dimension", t.name.c_str());
            if (!c.get(t.type) || !c.get(t.offset))
                return fail("tensor '%s': truncated entry", t.name.c_str());
            // element count and byte size, overflow-checked
            uint64_t elems = 1;
            for (uint32_t d = 0; d < t.n_dims; ++d)
            {
                if (t.dims[d] > UINT64_MAX / elems)
                    return fail("tensor '%s': element count overflows", t.name.c_str());
                elems *= t.dims[d];
            }
            const TypeSize ts = type_size(t.type);
            t.nbytes = 0;
            if (ts.block_bytes)
            {
                if (t.dims[0] % ts.block_elems)
                    return fail("tensor '%s': row length %llu is not a multiple of the block size %u", t.name.c_str(),
                                (unsigned long long)t.dims[0], ts.block_elems);
                const uint64_t blocks = elems / ts.block_elems;
                if (blocks > UINT64_MAX / ts.block_bytes)
                    return fail("tensor '%s': byte size overflows", t.name.c_str());
                t.nbytes = blocks * ts.block_bytes;
            }
            if (g.by_name.count(t.name))
                return fail("tensor '%s' appears twice", t.name.c_str());
            g.by_name.emplace(t.name, g.tensors.size());
            g.tensors.push_back(std::move(t));
        }
        uint64_t align = 32;
        auto it = g.meta.find("general.alignment");
        if (it != g.meta.end() && it->second.type != GV_STRING)
            align = it->second.bits;
        if (align == 0 || (align & (align - 1)) != 0 || align > (1u << 20))
            return fail("general.alignment=%llu is not a power of two up to 1 MiB", (unsigned long long)align);
        g.data_start = (c.at + align - 1) / align * align;
        if (g.data_start > g.size && !g.tensors.empty())
            return fail("no data section");
        for (const Tensor &t : g.tensors)
        {
            if (t.offset % align)
                return fail("tensor '%s': offset %llu is not aligned to %llu", t.name.c_str(),
                            (unsigned long long)t.offset, (unsigned long long)align);
            const uint64_t room = g.size - g.data_start;
            if (t.offset > room || t.nbytes > room - t.offset)
                return fail("tensor '%s' (%llu bytes at offset %llu) runs past the end of the file", t.name.c_str(),
                            (unsigned long long)t.nbytes, (unsigned long long)t.offset);
        }
        return true;
    }

    void fill(const Gguf &g, const Tensor &t, llam_gguf_tensor *out)
    {
        out->name = t.name.c_str();
        out->ggml_type = t.type;
        out->fmt = type_fmt(t.type);
        out->n_dims = t.n_dims;
        for (int d = 0; d < 4; ++d)
            out->dims[d] = t.dims[d];
        out->nbytes = t.nbytes;
        out->data = g.base + g.data_start + t.offset;
    }

    const MetaValue *meta_of(const void *gguf, const char *key)
    {
        if (!gguf || !key)
        {
            fail("null argument");
            return nullptr;
        }
        const Gguf *g = static_cast<const Gguf *>(gguf);
        auto it = g->meta.find(key);
        if (it == g->meta.end())
        {
            fail("no metadata key '%s'", key);
            return nullptr;
        }
        return &it->second;
    }

    // ---- container ------------------------------------------------------------------------
    static_assert(sizeof(llam_prepared_header) == 64, "the header is 64 bytes on disk");

    bool header_fields_ok(const llam_prepared_header &h)
    {
        if (h.magic != LLAM_PREPARED_MAGIC)
            return fail("not a prepared-weights file (magic)");
        if (h.version != LLAM_PREPARED_VERSION)
            return fail("container version %u, this library reads %u", h.version, LLAM_PREPARED_VERSION);
        const size_t bb = llam_format_block_bytes(h.fmt);
        if (bb == 0)
            return fail("unknown weight format %d", (int)h.fmt);
        if (h.N < 1 || h.K < 256 || (h.K % 256) != 0)
            return fail("bad shape %d x %d", h.N, h.K);
        if (h.block_bytes != bb)
            return fail("block size %u does not belong to format %d", h.block_bytes, (int)h.fmt);
        if (h.gguf_bytes != (uint64_t)h.N * (uint64_t)(h.K / 256) * bb)
            return fail("source size does not match the shape");
        if (h.prepared_bytes != (uint64_t)llam_ql_prepared_bytes(h.fmt, h.N, h.K))
            return fail("payload size %llu is not that of a prepared %d x %d matrix of format %d",
                        (unsigned long long)h.prepared_bytes, h.N, h.K, (int)h.fmt);
        for (uint8_t b : h.reserved0)
            if (b)
                return fail("reserved header bytes are not zero");
        for (uint8_t b : h.reserved1)
            if (b)
                return fail("reserved header bytes are not zero");
        return true;
    }

    struct File
    {
        FILE *f = nullptr;
        ~File()
        {
            if (f)
                fclose(f);
        }
    };
} // namespace

extern "C" const char *llam_weights_last_error(void) { return g_error; }

extern "C" void *llam_gguf_open(const char *path)
{
    if (!path)
    {
        fail("null path");
        return nullptr;
    }
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0)
    {
        fail("cannot open '%s'", path);
        return nullptr;
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 24)
    {
        close(fd);
        fail("'%s' is too short for a GGUF header", path);
        return nullptr;
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED)
    {
        fail("cannot map '%s'", path);
        return nullptr;
    }
    Gguf *g = new Gguf;
    g->base = static_cast<const uint8_t *>(map);
    g->size = (uint64_t)st.st_size;
    if (!parse(*g))
    {
        delete g;
        return nullptr;
    }
    return g;
}

extern "C" void llam_gguf_close(void *gguf) { delete static_cast<Gguf *>(gguf); }

extern "C" uint64_t llam_gguf_tensor_count(const void *gguf)
{
    return gguf ? static_cast<const Gguf *>(gguf)->tensors.size() : 0;
}

extern "C" bool llam_gguf_tensor_at(const void *gguf, uint64_t index, llam_gguf_tensor *out)
{
    if (!gguf || !out)
        return fail("null argument");
    const Gguf *g = static_cast<const Gguf *>(gguf);
    if (index >= g->tensors.size())
        return fail("tensor index %llu of %zu", (unsigned long long)index, g->tensors.size());
    fill(*g, g->tensors[(size_t)index], out);
    return true;
}

extern "C" bool llam_gguf_find(const void *gguf, const char *name, llam_gguf_tensor *out)
{
    if (!gguf || !name || !out)
        return fail("null argument");
    const Gguf *g = static_cast<const Gguf *>(gguf);
    auto it = g->by_name.find(name);
    if (it == g->by_name.end())
        return fail("no tensor '%s'", name);
    fill(*g, g->tensors[it->second], out);
    return true;
}

extern "C" bool llam_gguf_meta_u64(const void *gguf, const char *key, uint64_t *out)
{
    const MetaValue *v = meta_of(gguf, key);
    if (!v || !out)
        return v ? fail("null argument") : false;
    switch (v->type)
    {
    case GV_U8: case GV_U16: case GV_U32: case GV_U64: case GV_BOOL: *out = v->bits; return true;
    case GV_I8: *out = (uint64_t)(int64_t)(int8_t)v->bits; break;
    case GV_I16: *out = (uint64_t)(int64_t)(int16_t)v->bits; break;
    case GV_I32: *out = (uint64_t)(int64_t)(int32_t)v->bits; break;
    case GV_I64: *out = v->bits; break;
    default: return fail("metadata key '%s' is not an integer", key);
    }
    if ((int64_t)*out < 0)
        return fail("metadata key '%s' is negative", key);
    return true;
}

extern "C" bool llam_gguf_meta_f64(const void *gguf, const char *key, double *out)
{
    const MetaValue *v = meta_of(gguf, key);
    if (!v || !out)
        return v ? fail("null argument") : false;
    if (v->type == GV_F32)
    {
        float f;
        const uint32_t b = (uint32_t)v->bits;
        memcpy(&f, &b, 4);
        *out = f;
        return true;
    }
    if (v->type == GV_F64)
    {
        memcpy(out, &v->bits, 8);
        return true;
    }
    return fail("metadata key '%s' is not a float", key);
}

extern "C" const char *llam_gguf_meta_str(const void *gguf, const char *key)
{
    const MetaValue *v = meta_of(gguf, key);
    if (!v)
        return nullptr;
    if (v->type != GV_STRING)
    {
        fail("metadata key '%s' is not a string", key);
        return nullptr;
    }
    return v->str.c_str();
}

extern "C" uint64_t llam_weights_checksum(const void *bytes, uint64_t n)
{
    const uint8_t *p = static_cast<const uint8_t *>(bytes);
    uint64_t h = 0xcbf29ce484222325ull;
    uint64_t i = 0;
    for (; i + 8 <= n; i += 8)
    {
        uint64_t w;
        memcpy(&w, p + i, 8);
        h = (h ^ w) * 0x100000001b3ull;
    }
    if (i < n)
    {
        uint64_t w = 0;
        memcpy(&w, p + i, (size_t)(n - i));
        h = (h ^ w) * 0x100000001b3ull;
    }
    return h;
}

extern "C" bool llam_prepared_header_build(uint8_t fmt, int N, int K, const void *payload, llam_prepared_header *out)
{
    if (!out || !payload)
        return fail("null argument");
    const size_t bb = llam_format_block_bytes(fmt);
    if (bb == 0)
        return fail("unknown weight format %d", (int)fmt);
    if (N < 1 || K < 256 || (K % 256) != 0)
        return fail("bad shape %d x %d", N, K);
    memset(out, 0, sizeof *out);
    out->magic = LLAM_PREPARED_MAGIC;
    out->version = LLAM_PREPARED_VERSION;
    out->fmt = fmt;
    out->N = N;
    out->K = K;
    out->block_bytes = (uint32_t)bb;
    out->prepared_bytes = llam_ql_prepared_bytes(fmt, N, K);
    out->gguf_bytes = (uint64_t)N * (uint64_t)(K / 256) * bb;
    out->checksum = llam_weights_checksum(payload, out->prepared_bytes);
    return true;
}

extern "C" bool llam_prepared_buffer_check(const void *buffer, uint64_t buffer_bytes, bool verify_checksum)
{
    if (!buffer)
        return fail("null argument");
    if (buffer_bytes < sizeof(llam_prepared_header))
        return fail("buffer of %llu bytes is shorter than the header", (unsigned long long)buffer_bytes);
    llam_prepared_header h;
    memcpy(&h, buffer, sizeof h);
    if (!header_fields_ok(h))
        return false;
    if (h.prepared_bytes > buffer_bytes - sizeof h)
        return fail("payload of %llu bytes does not fit a buffer of %llu", (unsigned long long)h.prepared_bytes,
                    (unsigned long long)buffer_bytes);
    if (verify_checksum &&
        llam_weights_checksum(static_cast<const uint8_t *>(buffer) + sizeof h, h.prepared_bytes) != h.checksum)
        return fail("checksum mismatch: the payload is damaged");
    return true;
}

extern "C" bool llam_prepared_save(const char *path, uint8_t fmt, int N, int K, const void *d_prepared, int device_id)
{
    if (!path || !d_prepared)
        return fail("null argument");
    const size_t bytes = llam_ql_prepared_bytes(fmt, N, K);
    if (bytes == 0)
        return fail("format %d, shape %d x %d: nothing to save", (int)fmt, N, K);
    if (hipSetDevice(device_id) != hipSuccess)
        return fail("no HIP device %d", device_id);
    std::vector<uint8_t> host(bytes);
    if (hipMemcpy(host.data(), d_prepared, bytes, hipMemcpyDeviceToHost) != hipSuccess)
        return fail("copy of %zu bytes from the device failed", bytes);
    llam_prepared_header h;
    if (!llam_prepared_header_build(fmt, N, K, host.data(), &h))
        return false;
    File out;
    out.f = fopen(path, "wb");
    if (!out.f)
        return fail("cannot create '%s'", path);
    if (fwrite(&h, sizeof h, 1, out.f) != 1 || fwrite(host.data(), 1, bytes, out.f) != bytes || fflush(out.f) != 0)
        return fail("write to '%s' failed", path);
    return true;
}

extern "C" bool llam_prepared_load(const char *path, llam_prepared_header *out, void *d_prepared, uint64_t capacity,
                                   int device_id)
{
    if (!path || !out)
        return fail("null argument");
    File in;
    in.f = fopen(path, "rb");
    if (!in.f)
        return fail("cannot open '%s'", path);
    struct stat st;
    if (fstat(fileno(in.f), &st) != 0)
        return fail("cannot stat '%s'", path);
    llam_prepared_header h;
    if (fread(&h, sizeof h, 1, in.f) != 1)
        return fail("'%s' is shorter than the header", path);
    if (!header_fields_ok(h))
        return false;
    if ((uint64_t)st.st_size < sizeof h || h.prepared_bytes > (uint64_t)st.st_size - sizeof h)
        return fail("'%s' holds less than its header promises", path);
    *out = h;
    if (!d_prepared)
        return true;
    if (capacity < h.prepared_bytes)
        return fail("destination of %llu bytes is smaller than the payload of %llu", (unsigned long long)capacity,
                    (unsigned long long)h.prepared_bytes);
    std::vector<uint8_t> host((size_t)h.prepared_bytes);
    if (fread(host.data(), 1, host.size(), in.f) != host.size())
        return fail("read of '%s' failed", path);
    if (llam_weights_checksum(host.data(), host.size()) != h.checksum)
        return fail("checksum mismatch: '%s' is damaged", path);
    if (hipSetDevice(device_id) != hipSuccess)
        return fail("no HIP device %d", device_id);
    if (hipMemcpy(d_prepared, host.data(), host.size(), hipMemcpyHostToDevice) != hipSuccess)
        return fail("copy of %zu bytes to the device failed", host.size());
    return true;
}
