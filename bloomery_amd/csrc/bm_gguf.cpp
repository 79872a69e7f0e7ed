// A GGUF reader for the expert stacks of a model file: header, key-values, tensor table, and a tensor's bytes in a
// read-only mapping. The subset of the reference's reader (crates/gguf/src/lib.rs: Gguf::open :319, find :540,
// data :557, TensorInfo :103, value :439) that the MoE path's caller needs to hand a file's blocks to
// bm_weights_create: the block bytes on disk are the bytes the kernels read (crates/gpu/src/weights.rs:69-86).
// Host code only. A file is foreign input: every length, count and offset is checked against the mapping before it
// is used, sizes are computed with overflow checks, and a refusal names what it met.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/bm_moe.h"

namespace {

// ggml type table for the types a model file of this path holds: values a block, bytes a block
// (crates/gguf/src/lib.rs:1362 ggml_type_info; crates/gguf/src/qtype.rs).
struct TypeInfo {
    uint32_t id;
    uint64_t blck, size;
};
const TypeInfo kTypes[] = {
    {0, 1, 4},      // F32
    {1, 1, 2},      // F16
    {2, 32, 18},    // Q4_0
    {3, 32, 20},    // Q4_1
    {6, 32, 22},    // Q5_0
    {7, 32, 24},    // Q5_1
    {8, 32, 34},    // Q8_0
    {10, 256, 84},  // Q2_K
    {11, 256, 110}, // Q3_K
    {12, 256, 144}, // Q4_K
    {13, 256, 176}, // Q5_K
    {14, 256, 210}, // Q6_K
    {16, 256, 66},  // IQ2_XXS
    {17, 256, 74},  // IQ2_XS
    {18, 256, 98},  // IQ3_XXS
    {19, 256, 50},  // IQ1_S
    {20, 32, 18},   // IQ4_NL
    {21, 256, 110}, // IQ3_S
    {22, 256, 82},  // IQ2_S
    {23, 256, 136}, // IQ4_XS
    {24, 1, 1},     // I8
    {25, 1, 2},     // I16
    {26, 1, 4},     // I32
    {27, 1, 8},     // I64
    {28, 1, 8},     // F64
    {29, 256, 56},  // IQ1_M
    {30, 1, 2},     // BF16
};

const TypeInfo *type_info(uint32_t id) {
    for (const TypeInfo &t : kTypes)
        if (t.id == id) return &t;
    return nullptr;
}

struct Value {
    uint32_t type = 0;       // the file's value type id
    uint64_t bits = 0;       // integers, bool, f32 / f64 bit patterns
    std::string str;         // type 8
    uint32_t elem_type = 0;  // type 9: element type and count (the elements are skipped, not kept)
    uint64_t count = 0;
};

thread_local std::string g_gguf_err;

int refuse(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_gguf_err = buf;
    return code;
}

// A cursor over the mapping that refuses to step past its end.
struct Reader {
    const uint8_t *base;
    uint64_t len, at = 0;
    bool take(void *dst, uint64_t n) {
        if (n > len - at) return false;
        memcpy(dst, base + at, n);
        at += n;
        return true;
    }
    template <class T>
    bool get(T &v) {
        return take(&v, sizeof v);
    }
    bool skip(uint64_t n) {
        if (n > len - at) return false;
        at += n;
        return true;
    }
    bool string(std::string &s, uint64_t max_len) {
        uint64_t n;
        if (!get(n) || n > max_len || n > len - at) return false;
        s.assign(reinterpret_cast<const char *>(base + at), (size_t)n);
        at += n;
        return true;
    }
};

uint64_t scalar_size(uint32_t type) {
    switch (type) {
    case 0: case 1: case 7: return 1;
    case 2: case 3: return 2;
    case 4: case 5: case 6: return 4;
    case 10: case 11: case 12: return 8;
    default: return 0;
    }
}

bool checked_mul(uint64_t a, uint64_t b, uint64_t &out) { return !__builtin_mul_overflow(a, b, &out); }

} // namespace

struct bm_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    uint64_t len = 0;
    uint32_t version = 0;
    uint64_t alignment = 32, data_base = 0;
    std::vector<std::pair<std::string, Value>> kv;
    std::vector<bm_gguf_tensor> tensors;
    std::vector<std::string> names;
    std::unordered_map<std::string, size_t> by_name;
    std::vector<bm_gguf *> more; // the other shards of a split set, owned by the first
};

extern "C" {

const char *bm_gguf_last_error(void) { return g_gguf_err.c_str(); }

void bm_gguf_close(bm_gguf *g) {
    if (!g) return;
    for (bm_gguf *shard : g->more) bm_gguf_close(shard);
    if (g->map) munmap(const_cast<uint8_t *>(g->map), (size_t)g->len);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

} // extern "C"

// One file.
static int open_one(const char *path, bm_gguf **out) {
    *out = nullptr;
    bm_gguf *g = new (std::nothrow) bm_gguf;
    if (!g) return refuse(BM_EDRIVER, "bm_gguf_open: out of host memory");
    auto fail = [&](int code) {
        bm_gguf_close(g);
        return code;
    };
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    if (g->fd < 0) return fail(refuse(BM_EARG, "bm_gguf_open: cannot open %s", path));
    struct stat st;
    if (fstat(g->fd, &st) != 0 || st.st_size < 24) return fail(refuse(BM_ESHAPE, "bm_gguf_open: %s is shorter than a GGUF header", path));
    g->len = (uint64_t)st.st_size;
    void *m = mmap(nullptr, (size_t)g->len, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) return fail(refuse(BM_EDRIVER, "bm_gguf_open: cannot map %s", path));
    g->map = static_cast<const uint8_t *>(m);
    Reader r{g->map, g->len};
    uint32_t magic = 0;
    uint64_t n_tensors = 0, n_kv = 0;
    r.get(magic);
    r.get(g->version);
    if (magic != 0x46554747u) return fail(refuse(BM_ESHAPE, "bm_gguf_open: %s does not start with GGUF", path));
    if (g->version != 2 && g->version != 3)
        return fail(refuse(BM_ESHAPE, "bm_gguf_open: GGUF version %u (2 and 3 are read)", g->version));
    if (!r.get(n_tensors) || !r.get(n_kv)) return fail(refuse(BM_ESHAPE, "bm_gguf_open: the header ends early"));
    // a key-value or a tensor entry takes at least 12 bytes: counts past that are not this file's
    if (n_kv > g->len / 12 || n_tensors > g->len / 12)
        return fail(refuse(BM_ESHAPE, "bm_gguf_open: %llu key-values and %llu tensors in %llu bytes", (unsigned long long)n_kv,
                           (unsigned long long)n_tensors, (unsigned long long)g->len));
    for (uint64_t i = 0; i < n_kv; i++) {
        std::string key;
        Value v;
        if (!r.string(key, 1 << 16) || !r.get(v.type)) return fail(refuse(BM_ESHAPE, "bm_gguf_open: key-value %llu ends early", (unsigned long long)i));
        bool ok = true;
        if (v.type == 8) {
            ok = r.string(v.str, g->len);
        } else if (v.type == 9) {
            ok = r.get(v.elem_type) && r.get(v.count);
            if (ok && v.elem_type == 8) {
                std::string skip;
                for (uint64_t e = 0; ok && e < v.count; e++) ok = r.string(skip, g->len);
            } else if (ok) {
                uint64_t sz = scalar_size(v.elem_type), bytes;
                ok = sz != 0 && checked_mul(sz, v.count, bytes) && r.skip(bytes);
            }
        } else {
            const uint64_t sz = scalar_size(v.type);
            ok = sz != 0 && r.take(&v.bits, sz);
        }
        if (!ok) return fail(refuse(BM_ESHAPE, "bm_gguf_open: the value of %s (type %u) is not readable", key.c_str(), v.type));
        if (key == "general.alignment") {
            if ((v.type != 4 && v.type != 10) || v.bits == 0 || (v.bits & (v.bits - 1)) != 0 || v.bits > (1u << 20))
                return fail(refuse(BM_ESHAPE, "bm_gguf_open: general.alignment is not a power of two of a sane size"));
            g->alignment = v.bits;
        }
        g->kv.emplace_back(std::move(key), std::move(v));
    }
    g->tensors.reserve((size_t)n_tensors);
    g->names.reserve((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; i++) {
        std::string name;
        bm_gguf_tensor t;
        memset(&t, 0, sizeof t);
        uint32_t n_dims = 0;
        if (!r.string(name, 1 << 16) || !r.get(n_dims) || n_dims < 1 || n_dims > 4)
            return fail(refuse(BM_ESHAPE, "bm_gguf_open: tensor %llu's entry is not readable", (unsigned long long)i));
        t.n_dims = (int)n_dims;
        for (int d = 0; d < 4; d++) t.dims[d] = 1;
        bool ok = true;
        for (uint32_t d = 0; ok && d < n_dims; d++) ok = r.get(t.dims[d]) && t.dims[d] > 0;
        uint32_t type = 0;
        ok = ok && r.get(type) && r.get(t.offset);
        if (!ok) return fail(refuse(BM_ESHAPE, "bm_gguf_open: tensor %s's entry is not readable", name.c_str()));
        t.type = (int)type;
        const TypeInfo *ti = type_info(type);
        if (ti) { // the contiguous size: type_size * (ne0 / blck) * ne1 * ...
            uint64_t n = 0;
            ok = t.dims[0] % ti->blck == 0 && checked_mul(t.dims[0] / ti->blck, ti->size, n);
            for (uint32_t d = 1; ok && d < n_dims; d++) ok = checked_mul(n, t.dims[d], n);
            if (!ok) return fail(refuse(BM_ESHAPE, "bm_gguf_open: tensor %s's dimensions do not size in its type %u", name.c_str(), type));
            t.nbytes = n;
        } else {
            t.nbytes = 0; // a type this table does not hold: listed, never handed out
        }
        if (t.offset % g->alignment != 0)
            return fail(refuse(BM_ESHAPE, "bm_gguf_open: tensor %s sits at offset %llu, off the file's alignment %llu", name.c_str(),
                               (unsigned long long)t.offset, (unsigned long long)g->alignment));
        if (g->by_name.count(name)) return fail(refuse(BM_ESHAPE, "bm_gguf_open: two tensors are named %s", name.c_str()));
        g->by_name.emplace(name, g->tensors.size());
        g->names.push_back(std::move(name));
        g->tensors.push_back(t);
    }
    g->data_base = (r.at + g->alignment - 1) / g->alignment * g->alignment;
    if (g->data_base > g->len && !g->tensors.empty())
        return fail(refuse(BM_ESHAPE, "bm_gguf_open: the data section starts past the end of the file"));
    for (size_t i = 0; i < g->tensors.size(); i++) {
        bm_gguf_tensor &t = g->tensors[i];
        t.name = g->names[i].c_str();
        uint64_t start = 0, end = 0;
        if (__builtin_add_overflow(g->data_base, t.offset, &start) || __builtin_add_overflow(start, t.nbytes, &end) || end > g->len)
            return fail(refuse(BM_ESHAPE, "bm_gguf_open: tensor %s (%llu bytes at %llu + %llu) runs past the file's %llu bytes", t.name,
                               (unsigned long long)t.nbytes, (unsigned long long)g->data_base, (unsigned long long)t.offset,
                               (unsigned long long)g->len));
        t.data = t.nbytes ? g->map + start : nullptr;
    }
    *out = g;
    return BM_OK;
}

static const Value *value_of(const bm_gguf *g, const char *key);

// A split key as a count (llama.cpp's splitter writes split.no and split.count as u16, split.tensors.count as i32).
static bool split_count(const bm_gguf *g, const char *key, uint64_t *out) {
    const Value *v = value_of(g, key);
    if (!v) return false;
    switch (v->type) {
    case 0: case 2: case 4: case 10: // u8, u16, u32, u64
        *out = v->bits;
        return true;
    case 1: case 3: case 5: case 11: { // i8, i16, i32, i64: a count is not negative
        const uint64_t sz = scalar_size(v->type);
        const int64_t sv = (int64_t)(v->bits << (64 - 8 * sz)) >> (64 - 8 * sz);
        if (sv < 0) return false;
        *out = (uint64_t)sv;
        return true;
    }
    default:
        return false;
    }
}

extern "C" {

// One file, whatever split keys it holds (crates/gguf/src/lib.rs:359 Gguf::open_split_shard reads one shard so).
int bm_gguf_open(const char *path, bm_gguf **out) {
    if (!path || !out) return refuse(BM_EARG, "bm_gguf_open: NULL argument");
    return open_one(path, out);
}

// A model as one file or as llama.cpp's split set named by its first shard (crates/gguf/src/lib.rs:835-875
// Split::open_model): a file without split.count is a set of one. Otherwise split.count is a count above 0, the first
// file's split.no is 0, a set of several is named <prefix>-00001-of-%05d.gguf and its siblings
// <prefix>-%05d-of-%05d.gguf all open, every shard's split.no is its place, every split.count agrees, the shards'
// tensor counts sum to the first shard's split.tensors.count and no tensor name appears twice, or the set is refused.
// The metadata is the first shard's: the splitter writes the model's keys there alone.
int bm_gguf_open_split(const char *first, bm_gguf **out) {
    if (!first || !out) return refuse(BM_EARG, "bm_gguf_open_split: NULL argument");
    bm_gguf *g = nullptr;
    int rc = open_one(first, &g);
    *out = nullptr;
    if (rc) return rc;
    if (!value_of(g, "split.count")) {
        *out = g;
        return BM_OK;
    }
    auto fail = [&](int code) {
        bm_gguf_close(g);
        return code;
    };
    auto place_of = [&](const bm_gguf *shard, const char *path, uint64_t place) {
        uint64_t no = 0;
        if (!split_count(shard, "split.no", &no)) return refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.no is absent or not a count", path);
        if (no != place)
            return refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.no is %llu, but the file is shard %llu of its set (from 0)", path,
                          (unsigned long long)no, (unsigned long long)place);
        return (int)BM_OK;
    };
    uint64_t count = 0;
    if (!split_count(g, "split.count", &count) || count == 0 || count > 99999)
        return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.count is not a count from 1 to 99999", first));
    if ((rc = place_of(g, first, 0)) != BM_OK) return fail(rc);
    uint64_t seen = g->tensors.size();
    if (count > 1) {
        char suffix[32];
        snprintf(suffix, sizeof suffix, "-%05d-of-%05d.gguf", 1, (int)count);
        const std::string name(first);
        const size_t ns = strlen(suffix);
        if (name.size() <= ns || name.compare(name.size() - ns, ns, suffix) != 0)
            return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: %s holds split.count = %llu, but its name does not end in %s", first,
                               (unsigned long long)count, suffix));
        const std::string prefix = name.substr(0, name.size() - ns);
        for (uint64_t i = 1; i < count; i++) {
            snprintf(suffix, sizeof suffix, "-%05d-of-%05d.gguf", (int)i + 1, (int)count);
            const std::string sib = prefix + suffix;
            bm_gguf *shard = nullptr;
            rc = open_one(sib.c_str(), &shard);
            if (rc) {
                const std::string why = g_gguf_err; // names the shard's file
                return fail(refuse(rc, "bm_gguf_open_split: shard %llu of %llu: %s", (unsigned long long)i + 1, (unsigned long long)count, why.c_str()));
            }
            g->more.push_back(shard);
            if ((rc = place_of(shard, sib.c_str(), i)) != BM_OK) return fail(rc);
            uint64_t theirs = 0;
            if (!split_count(shard, "split.count", &theirs) || theirs != count)
                return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.count is not the first shard's %llu", sib.c_str(), (unsigned long long)count));
            seen += shard->tensors.size();
        }
    }
    uint64_t want = 0;
    if (!split_count(g, "split.tensors.count", &want))
        return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.tensors.count is absent or not a count", first));
    if (seen != want)
        return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: %s: split.tensors.count is %llu, but the %llu shards hold %llu tensors", first,
                           (unsigned long long)want, (unsigned long long)count, (unsigned long long)seen));
    // the set's tensors behind the first shard's: an entry's name and data point into its own shard, which g owns
    for (bm_gguf *shard : g->more) {
        for (size_t t = 0; t < shard->tensors.size(); t++) {
            const std::string &tn = shard->names[t];
            if (g->by_name.count(tn)) return fail(refuse(BM_ESHAPE, "bm_gguf_open_split: tensor %s is in two shards of the set", tn.c_str()));
            g->by_name.emplace(tn, g->tensors.size());
            g->tensors.push_back(shard->tensors[t]);
        }
    }
    *out = g;
    return BM_OK;
}

int bm_gguf_version(const bm_gguf *g) { return g ? (int)g->version : 0; }
int64_t bm_gguf_tensor_count(const bm_gguf *g) { return g ? (int64_t)g->tensors.size() : 0; }

int bm_gguf_tensor_at(const bm_gguf *g, int64_t i, bm_gguf_tensor *out) {
    if (!g || !out) return refuse(BM_EARG, "bm_gguf_tensor_at: NULL argument");
    if (i < 0 || (size_t)i >= g->tensors.size())
        return refuse(BM_ESHAPE, "bm_gguf_tensor_at: tensor %lld of %zu", (long long)i, g->tensors.size());
    *out = g->tensors[(size_t)i];
    return BM_OK;
}

int bm_gguf_find(const bm_gguf *g, const char *name, bm_gguf_tensor *out) {
    if (!g || !name || !out) return refuse(BM_EARG, "bm_gguf_find: NULL argument");
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) return refuse(BM_ESHAPE, "bm_gguf_find: the file holds no tensor named %s", name);
    *out = g->tensors[it->second];
    return BM_OK;
}

static const Value *value_of(const bm_gguf *g, const char *key) {
    for (const auto &kv : g->kv)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

int bm_gguf_get_u64(const bm_gguf *g, const char *key, uint64_t *out) {
    if (!g || !key || !out) return refuse(BM_EARG, "bm_gguf_get_u64: NULL argument");
    const Value *v = value_of(g, key);
    if (!v) return refuse(BM_ESHAPE, "bm_gguf_get_u64: the file holds no key %s", key);
    switch (v->type) { // the unsigned types, and the signed ones when not negative (crates/gguf/src/lib.rs:1510 as_u64)
    case 0: case 2: case 4: case 10: case 7: *out = v->bits; return BM_OK;
    case 1: if ((int8_t)v->bits >= 0) { *out = (uint64_t)(int8_t)v->bits; return BM_OK; } break;
    case 3: if ((int16_t)v->bits >= 0) { *out = (uint64_t)(int16_t)v->bits; return BM_OK; } break;
    case 5: if ((int32_t)v->bits >= 0) { *out = (uint64_t)(int32_t)v->bits; return BM_OK; } break;
    case 11: if ((int64_t)v->bits >= 0) { *out = v->bits; return BM_OK; } break;
    default: break;
    }
    return refuse(BM_ETYPE, "bm_gguf_get_u64: %s holds a value of type %u, not a count", key, v->type);
}

int bm_gguf_get_f32(const bm_gguf *g, const char *key, float *out) {
    if (!g || !key || !out) return refuse(BM_EARG, "bm_gguf_get_f32: NULL argument");
    const Value *v = value_of(g, key);
    if (!v) return refuse(BM_ESHAPE, "bm_gguf_get_f32: the file holds no key %s", key);
    if (v->type != 6) return refuse(BM_ETYPE, "bm_gguf_get_f32: %s holds a value of type %u, not an f32", key, v->type);
    const uint32_t bits = (uint32_t)v->bits;
    memcpy(out, &bits, 4);
    return BM_OK;
}

const char *bm_gguf_get_str(const bm_gguf *g, const char *key) {
    if (!g || !key) return nullptr;
    const Value *v = value_of(g, key);
    return v && v->type == 8 ? v->str.c_str() : nullptr;
}

} // extern "C"
