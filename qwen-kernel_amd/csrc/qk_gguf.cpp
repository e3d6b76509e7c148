// qk_gguf.cpp -- read-only GGUF reader behind include/qk_gguf.h (host code, no GPU calls).
// File format as the reference reads it (src/gguf.h:112-197): magic "GGUF", u32 version (>= 2),
// u64 tensor count, u64 KV count, the KVs (string key, u32 type, value), the tensor infos (name,
// u32 n_dims, u64 dims, u32 type, u64 offset) and, aligned to general.alignment (default 32), the
// data section.  A cursor that refuses to move past the end of the mapping replaces the
// reference's unchecked reads.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/qk_gguf.h"
#include "qk_host.h"

namespace {

using qk::fail;

struct Shard {
    const uint8_t* base = nullptr;
    size_t size = 0;
};

struct Tensor {
    std::string name;
    uint32_t type = 0, n_dims = 0, shard = 0;
    uint64_t ne[4] = {1, 1, 1, 1};
    const uint8_t* data = nullptr;
    uint64_t nbytes = 0;
};

// Reads little-endian scalars and length-prefixed strings; `ok` turns false, and stays false,
// at the first read that would leave the mapping.
struct Cursor {
    const uint8_t* base;
    size_t size, pos = 0;
    bool ok = true;
    template <typename T>
    T rd()
    {
        T v{};
        if (!ok || size - pos < sizeof(T)) { ok = false; return v; }
        memcpy(&v, base + pos, sizeof(T));
        pos += sizeof(T);
        return v;
    }
    std::string str()
    {
        const uint64_t n = rd<uint64_t>();
        if (!ok || n > size - pos) { ok = false; return std::string(); }
        std::string s((const char*)base + pos, (size_t)n);
        pos += (size_t)n;
        return s;
    }
    void skip(uint64_t n)
    {
        if (!ok || n > size - pos) { ok = false; return; }
        pos += (size_t)n;
    }
};

constexpr uint32_t KV_STRING = 8, KV_ARRAY = 9;

// bytes of a fixed-size KV scalar type, 0 for string / array / unknown (reference src/gguf.h:140-156)
uint32_t scalar_bytes(uint32_t t)
{
    switch (t) {
    case 0: case 1: case 7: return 1;
    case 2: case 3: return 2;
    case 4: case 5: case 6: return 4;
    case 10: case 11: case 12: return 8;
    default: return 0;
    }
}

} // namespace

struct qkg_file {
    std::vector<Shard> shards;
    std::map<std::string, Tensor> tensors;
    std::vector<const Tensor*> order; // name order, filled after the last shard
    std::map<std::string, uint64_t> kv_int;
    std::map<std::string, std::string> kv_str;
    uint32_t version = 0;
    uint64_t split_tensors_total = 0;

    ~qkg_file()
    {
        for (auto& s : shards)
            if (s.base) munmap((void*)s.base, s.size);
    }

    // Skips one value of type t; for integer scalars returns the value through *out.
    bool skip_value(Cursor& c, uint32_t t, uint64_t* out, int depth)
    {
        if (t == KV_STRING) { c.str(); return c.ok; }
        if (t == KV_ARRAY) {
            if (depth > 4) return false;
            const uint32_t et = c.rd<uint32_t>();
            const uint64_t n = c.rd<uint64_t>();
            if (!c.ok) return false;
            if (const uint32_t sb = scalar_bytes(et)) {
                if (n > (c.size - c.pos) / sb) return false;
                c.skip(n * sb);
                return c.ok;
            }
            if (et != KV_STRING && et != KV_ARRAY) return false;
            if (n > c.size - c.pos) return false; // every element takes at least one byte
            for (uint64_t i = 0; i < n; i++)
                if (!skip_value(c, et, nullptr, depth + 1)) return false;
            return true;
        }
        uint64_t v = 0;
        switch (t) {
        case 0: case 7: v = c.rd<uint8_t>(); break;
        case 1: v = (uint64_t)(int64_t)c.rd<int8_t>(); break;
        case 2: v = c.rd<uint16_t>(); break;
        case 3: v = (uint64_t)(int64_t)c.rd<int16_t>(); break;
        case 4: v = c.rd<uint32_t>(); break;
        case 5: v = (uint64_t)(int64_t)c.rd<int32_t>(); break;
        case 6: c.rd<uint32_t>(); break;  // f32: skipped
        case 10: v = c.rd<uint64_t>(); break;
        case 11: v = (uint64_t)c.rd<int64_t>(); break;
        case 12: c.rd<uint64_t>(); break; // f64: skipped
        default: return false;
        }
        if (out) *out = v;
        return c.ok;
    }

    int open_one(const std::string& path, uint32_t* split_count)
    {
        const int fd = ::open(path.c_str(), O_RDONLY);
        if (fd < 0) return fail(QKG_EIO, "gguf: %s: %s", path.c_str(), strerror(errno));
        struct stat st;
        if (fstat(fd, &st) != 0 || st.st_size < 0) {
            ::close(fd);
            return fail(QKG_EIO, "gguf: %s: stat failed", path.c_str());
        }
        const size_t size = (size_t)st.st_size;
        if (size < 24) {
            ::close(fd);
            return fail(QKG_EFORMAT, "gguf: %s: %zu bytes is too short for a header", path.c_str(), size);
        }
        void* m = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
        ::close(fd); // the mapping holds its own reference
        if (m == MAP_FAILED) return fail(QKG_EIO, "gguf: %s: mmap: %s", path.c_str(), strerror(errno));
        const uint32_t shard = (uint32_t)shards.size();
        shards.push_back(Shard{(const uint8_t*)m, size});

        Cursor c{(const uint8_t*)m, size};
        if (memcmp(c.base, "GGUF", 4) != 0) return fail(QKG_EFORMAT, "gguf: %s: not a GGUF file", path.c_str());
        c.pos = 4;
        const uint32_t ver = c.rd<uint32_t>();
        if (ver < 2 || ver > 3) return fail(QKG_EFORMAT, "gguf: %s: version %u unsupported", path.c_str(), ver);
        if (shard == 0) version = ver;
        const uint64_t n_tensors = c.rd<uint64_t>(), n_kv = c.rd<uint64_t>();
        // every KV and every tensor info takes more than 12 bytes: counts beyond that are corrupt
        if (n_tensors > size / 12 || n_kv > size / 12)
            return fail(QKG_EFORMAT, "gguf: %s: implausible counts (%llu tensors, %llu keys)", path.c_str(),
                        (unsigned long long)n_tensors, (unsigned long long)n_kv);
        uint64_t alignment = 32; // per shard (reference src/gguf.h:164)
        for (uint64_t i = 0; i < n_kv; i++) {
            const std::string key = c.str();
            const uint32_t t = c.rd<uint32_t>();
            if (!c.ok) break;
            if (t == KV_STRING) {
                const std::string v = c.str();
                if (c.ok && shard == 0) kv_str[key] = v;
                continue;
            }
            uint64_t v = 0;
            if (!skip_value(c, t, &v, 0))
                return fail(QKG_EFORMAT, "gguf: %s: bad value for key \"%s\" (type %u)", path.c_str(), key.c_str(), t);
            const bool is_int = t <= 5 || t == 7 || t == 10 || t == 11; // not f32 / f64 / array
            if (is_int && shard == 0) kv_int[key] = v;
            if (is_int && key == "general.alignment" && v) alignment = v;
            if (is_int && key == "split.count" && split_count) *split_count = (uint32_t)v;
            if (is_int && key == "split.tensors.count") split_tensors_total = v;
        }
        if (!c.ok) return fail(QKG_EFORMAT, "gguf: %s: truncated in the metadata", path.c_str());
        if (alignment == 0 || alignment > (1u << 20) || (alignment & (alignment - 1)))
            return fail(QKG_EFORMAT, "gguf: %s: general.alignment %llu is not a power of two", path.c_str(),
                        (unsigned long long)alignment);

        struct Info {
            Tensor t;
            uint64_t off;
        };
        std::vector<Info> infos;
        infos.reserve((size_t)n_tensors);
        for (uint64_t i = 0; i < n_tensors; i++) {
            Info inf;
            inf.t.name = c.str();
            inf.t.n_dims = c.rd<uint32_t>();
            if (!c.ok) break;
            if (inf.t.n_dims > 4)
                return fail(QKG_EFORMAT, "gguf: %s: tensor \"%s\" has %u dimensions", path.c_str(), inf.t.name.c_str(),
                            inf.t.n_dims);
            for (uint32_t d = 0; d < inf.t.n_dims; d++) inf.t.ne[d] = c.rd<uint64_t>();
            inf.t.type = c.rd<uint32_t>();
            inf.off = c.rd<uint64_t>();
            inf.t.shard = shard;
            infos.push_back(std::move(inf));
        }
        if (!c.ok) return fail(QKG_EFORMAT, "gguf: %s: truncated in the tensor directory", path.c_str());
        const uint64_t data_start = (c.pos + alignment - 1) / alignment * alignment;
        if (data_start > size && !infos.empty())
            return fail(QKG_EFORMAT, "gguf: %s: no data section", path.c_str());
        for (auto& inf : infos) {
            Tensor& t = inf.t;
            if (inf.off > size - data_start)
                return fail(QKG_EFORMAT, "gguf: %s: tensor \"%s\" starts beyond the file", path.c_str(), t.name.c_str());
            // bytes, where the row size of the type is known; overflow-checked
            const size_t rb = qkk_row_bytes((int)t.type, t.ne[0]);
            uint64_t rows = 1;
            bool overflow = false;
            for (int d = 1; d < 4; d++) {
                if (t.ne[d] && rows > UINT64_MAX / t.ne[d]) overflow = true;
                rows *= t.ne[d];
            }
            if (rb && (overflow || rows > UINT64_MAX / rb))
                return fail(QKG_EFORMAT, "gguf: %s: tensor \"%s\" has an impossible shape", path.c_str(), t.name.c_str());
            t.nbytes = rb ? rows * rb : 0;
            if (t.nbytes > size - data_start - inf.off)
                return fail(QKG_EFORMAT, "gguf: %s: tensor \"%s\" (%llu bytes) runs past the end of the file",
                            path.c_str(), t.name.c_str(), (unsigned long long)t.nbytes);
            t.data = c.base + data_start + inf.off;
            tensors[t.name] = t; // a later shard's tensor of the same name replaces the earlier one, as in the reference
        }
        return QKK_OK;
    }

    int open_all(const std::string& path)
    {
        uint32_t split_count = 0;
        if (int rc = open_one(path, &split_count)) return rc;
        if (split_count > 1) {
            // "<prefix>-00001-of-NNNNN.gguf" (reference src/gguf.h:66-85)
            static const char marker[] = "-00001-of-";
            const size_t tp = path.rfind(marker);
            const bool ok_name = tp != std::string::npos && path.size() == tp + 10 + 5 + 5 &&
                                 path.compare(path.size() - 5, 5, ".gguf") == 0;
            if (!ok_name)
                return fail(QKG_EFORMAT, "gguf: split.count=%u but %s is not a -00001-of-NNNNN.gguf first shard",
                            split_count, path.c_str());
            if (split_count > 99999) return fail(QKG_EFORMAT, "gguf: split.count=%u", split_count);
            const std::string prefix = path.substr(0, tp);
            for (uint32_t i = 2; i <= split_count; i++) {
                char name[64];
                snprintf(name, sizeof name, "-%05u-of-%05u.gguf", i, split_count);
                if (int rc = open_one(prefix + name, nullptr)) return rc;
            }
            if (split_tensors_total && tensors.size() != (size_t)split_tensors_total)
                return fail(QKG_EFORMAT, "gguf: split.tensors.count=%llu but the shards hold %zu tensors",
                            (unsigned long long)split_tensors_total, tensors.size());
        }
        order.reserve(tensors.size());
        for (auto& kv : tensors) order.push_back(&kv.second);
        return QKK_OK;
    }
};

namespace {

void export_tensor(const Tensor& t, qkg_tensor* out)
{
    out->name = t.name.c_str();
    out->type = t.type;
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) out->ne[d] = t.ne[d];
    out->data = t.data;
    out->nbytes = t.nbytes;
    out->shard = t.shard;
    out->pad = 0;
}

} // namespace

extern "C" {

qkg_file* qkg_open(const char* path)
{
    if (!path || !*path) {
        fail(QKK_EINVAL, "qkg_open: no path");
        return nullptr;
    }
    qkg_file* f = new qkg_file();
    if (f->open_all(path) != QKK_OK) {
        delete f;
        return nullptr;
    }
    return f;
}

void qkg_close(qkg_file* f) { delete f; }

uint32_t qkg_version(const qkg_file* f) { return f ? f->version : 0; }
uint32_t qkg_n_shards(const qkg_file* f) { return f ? (uint32_t)f->shards.size() : 0; }
uint64_t qkg_n_tensors(const qkg_file* f) { return f ? f->order.size() : 0; }

int qkg_tensor_at(const qkg_file* f, uint64_t i, qkg_tensor* out)
{
    if (!f || !out) return fail(QKK_EINVAL, "qkg_tensor_at: null pointer");
    if (i >= f->order.size()) return fail(QKG_ENOTFOUND, "qkg_tensor_at: index %llu of %zu", (unsigned long long)i, f->order.size());
    export_tensor(*f->order[(size_t)i], out);
    return QKK_OK;
}

int qkg_find(const qkg_file* f, const char* name, qkg_tensor* out)
{
    if (!f || !name || !out) return fail(QKK_EINVAL, "qkg_find: null pointer");
    const auto it = f->tensors.find(name);
    if (it == f->tensors.end()) return fail(QKG_ENOTFOUND, "gguf: no tensor \"%s\"", name);
    export_tensor(it->second, out);
    return QKK_OK;
}

int qkg_kv_int(const qkg_file* f, const char* key, uint64_t* out)
{
    if (!f || !key || !out) return fail(QKK_EINVAL, "qkg_kv_int: null pointer");
    const auto it = f->kv_int.find(key);
    if (it == f->kv_int.end()) return fail(QKG_ENOTFOUND, "gguf: no integer key \"%s\"", key);
    *out = it->second;
    return QKK_OK;
}

int qkg_kv_str(const qkg_file* f, const char* key, const char** out)
{
    if (!f || !key || !out) return fail(QKK_EINVAL, "qkg_kv_str: null pointer");
    const auto it = f->kv_str.find(key);
    if (it == f->kv_str.end()) return fail(QKG_ENOTFOUND, "gguf: no string key \"%s\"", key);
    *out = it->second.c_str();
    return QKK_OK;
}

int qkg_moe_layer(const qkg_file* f, uint32_t layer, qkg_moe_tensors* out)
{
    if (!f || !out) return fail(QKK_EINVAL, "qkg_moe_layer: null pointer");
    memset(out, 0, sizeof *out);
    struct Want {
        const char* suffix;
        qkg_tensor* dst;
    } want[8] = {{"ffn_gate_inp.weight", &out->gate_inp},     {"ffn_gate_inp_shexp.weight", &out->gate_inp_shexp},
                 {"ffn_gate_exps.weight", &out->gate_exps},   {"ffn_up_exps.weight", &out->up_exps},
                 {"ffn_down_exps.weight", &out->down_exps},   {"ffn_gate_shexp.weight", &out->gate_shexp},
                 {"ffn_up_shexp.weight", &out->up_shexp},     {"ffn_down_shexp.weight", &out->down_shexp}};
    for (auto& w : want) {
        char name[128];
        snprintf(name, sizeof name, "blk.%u.%s", layer, w.suffix);
        const auto it = f->tensors.find(name);
        if (it == f->tensors.end()) return fail(QKG_ENOTFOUND, "layer %u: missing MoE tensor %s", layer, name);
        export_tensor(it->second, w.dst);
    }
    // types (reference src/main.cpp:1283-1291; the IQ4_XS gate/up variant of the larger model is
    // not covered by the kernels here)
    if (out->gate_inp.type != QKK_F32 || out->gate_inp_shexp.type != QKK_F32 || out->gate_exps.type != QKK_IQ3_XXS ||
        out->up_exps.type != QKK_IQ3_XXS || (out->down_exps.type != QKK_IQ4_XS && out->down_exps.type != QKK_Q6_K) ||
        out->gate_shexp.type != QKK_Q8_0 || out->up_shexp.type != QKK_Q8_0 || out->down_shexp.type != QKK_Q8_0)
        return fail(QKK_ETYPE, "layer %u: unexpected MoE tensor types", layer);
    const uint64_t H = out->gate_exps.ne[0], F = out->gate_exps.ne[1], E = out->gate_exps.ne[2];
    if (H == 0 || F == 0 || E == 0 || H > 0xFFFFFFFFull || F > 0xFFFFFFFFull || E > QKK_MAX_EXPERTS)
        return fail(QKK_ESHAPE, "layer %u: gate_exps shape [%llu, %llu, %llu] is outside the kernels' limits", layer,
                    (unsigned long long)H, (unsigned long long)F, (unsigned long long)E);
    // top-k from the file (reference src/main.cpp:1295-1301)
    uint64_t n_used = 8;
    const auto arch = f->kv_str.find("general.architecture");
    const auto ku = f->kv_int.find((arch == f->kv_str.end() ? std::string() : arch->second) + ".expert_used_count");
    if (ku != f->kv_int.end()) n_used = ku->second;
    if (n_used < 1 || n_used > QKK_MAX_USED || n_used > E)
        return fail(QKK_ESHAPE, "layer %u: expert_used_count %llu unsupported", layer, (unsigned long long)n_used);
    // shapes of the other seven against gate_exps
    const auto shape = [](const qkg_tensor& t, uint64_t a, uint64_t b, uint64_t c) {
        return t.ne[0] == a && t.ne[1] == b && t.ne[2] == c && t.ne[3] == 1;
    };
    if (!shape(out->gate_exps, H, F, E) || !shape(out->up_exps, H, F, E) || !shape(out->down_exps, F, H, E) ||
        !shape(out->gate_inp, H, E, 1) || !shape(out->gate_inp_shexp, H, 1, 1) || !shape(out->gate_shexp, H, F, 1) ||
        !shape(out->up_shexp, H, F, 1) || !shape(out->down_shexp, F, H, 1))
        return fail(QKK_ESHAPE, "layer %u: MoE tensor shapes do not fit n_embd=%llu n_ff=%llu n_expert=%llu", layer,
                    (unsigned long long)H, (unsigned long long)F, (unsigned long long)E);
    for (auto& w : want)
        if (w.dst->nbytes == 0) return fail(QKK_ESHAPE, "layer %u: %s has a row length its type does not divide", layer, w.dst->name);
    out->n_embd = (uint32_t)H;
    out->n_ff = (uint32_t)F;
    out->n_expert = (uint32_t)E;
    out->n_used = (uint32_t)n_used;
    out->gu_type = (int32_t)out->gate_exps.type;
    out->down_type = (int32_t)out->down_exps.type;
    return QKK_OK;
}

} // extern "C"
