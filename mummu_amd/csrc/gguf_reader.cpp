// GGUF container reader and expert-bank locator (host only): header, typed metadata, tensor
// table, payload alignment and split shard sets, validated the way the reference validates them,
// so that the MoE blocks of a real OLMoE / Qwen-MoE file reach the kernels with zero repacking -
// the payload bytes of `blk.L.ffn_{gate,up,down}_exps.weight` and `blk.L.ffn_gate_inp.weight`
// are mapped and handed to mummu_moe_load_layer as they lie in the file.
//
// Reference behaviour followed (physics515/Mummu, crates/mummu/src/): gguf.rs:29-41 (bounds),
// :298-382 (type table), :473-513 (shard names), :577-714 (open, open_sharded), :1184-1376
// (values, header, tensor table, overlap check); models/olmoe.rs:116-179 (config keys),
// :325-347 (tensor names); models/qwen4exp/experts.rs:869-911 (bank locator and the
// geometry-versus-byte-length check).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/mummu_moe.h"

namespace {

constexpr uint64_t kMaxKvs = 4096, kMaxTensors = 65536, kMaxStringBytes = 1ull << 20, kMaxArrayLen = 1ull << 22;
constexpr uint32_t kMaxDims = 4;
constexpr uint64_t kDefaultAlignment = 32, kMaxShards = 64;

thread_local std::string g_gguf_error;

struct TypeInfo {
    uint32_t id;
    uint32_t block_size, block_bytes;
};
// ggml type id -> (elements per block, bytes per block); ids the reference knows (gguf.rs:298-382)
const TypeInfo kTypes[] = {{0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},   {6, 32, 22},   {7, 32, 24},
                           {8, 32, 34},    {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176},
                           {14, 256, 210}, {15, 256, 292}, {17, 256, 74},  {18, 256, 98},  {20, 32, 18},  {21, 256, 110},
                           {22, 256, 82},  {23, 256, 136}, {30, 1, 2},     {41, 128, 18},  {42, 64, 18},  {142, 128, 34},
                           {143, 128, 28}};

const TypeInfo *type_info(uint32_t id) {
    for (const TypeInfo &t : kTypes)
        if (t.id == id) return &t;
    return nullptr;
}

struct Value {
    uint32_t type = 0;  // GGUF value type id; arrays keep their items
    uint64_t u = 0;     // unsigned / bool
    int64_t i = 0;      // signed
    double f = 0.0;     // floats
    std::string s;
    std::vector<Value> items;
    // any unsigned integer type widened; signed, float and bool values are not integers here
    // (GgufValue::as_u64, gguf.rs:149-157)
    bool as_u64(uint64_t &out) const {
        if (type != 0 && type != 2 && type != 4 && type != 10) return false;
        out = u;
        return true;
    }
};

struct Tensor {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t type = 0;
    uint64_t offset = 0;  // relative to its own shard's payload base
    uint64_t nbytes = 0;
    int shard = 0;
};

struct Shard {
    std::string path;
    uint64_t data_offset = 0;
    int fd = -1;
    void *map = nullptr;
    size_t map_len = 0;
};

struct Parsed {
    uint32_t version = 0;
    uint64_t alignment = kDefaultAlignment, data_offset = 0;
    std::vector<std::pair<std::string, Value>> metadata;
    std::vector<Tensor> tensors;
};

int fail(int code, const std::string &msg) {
    g_gguf_error = msg;
    return code;
}

class Reader {
  public:
    Reader(FILE *f, std::string path) : f_(f), path_(std::move(path)) {}
    const std::string &path() const { return path_; }
    std::string err;
    int code = MUMMU_OK;

    bool bytes(void *dst, size_t n) {
        if (fread(dst, 1, n, f_) != n) return bad(MUMMU_ERR_IO, path_ + ": file ends inside the header");
        return true;
    }
    bool u32(uint32_t &v) { return bytes(&v, 4); }
    bool u64(uint64_t &v) { return bytes(&v, 8); }
    bool string(std::string &out, const char *what) {
        uint64_t len;
        if (!u64(len)) return false;
        if (len > kMaxStringBytes)
            return bad(MUMMU_ERR_GGUF, path_ + ": " + what + " of " + std::to_string(len) + " bytes exceeds the bound " + std::to_string(kMaxStringBytes));
        out.resize((size_t)len);
        if (len && !bytes(&out[0], (size_t)len)) return false;
        if (!valid_utf8(out)) return bad(MUMMU_ERR_GGUF, path_ + ": " + what + ": invalid UTF-8");
        return true;
    }
    bool value(const std::string &key, uint32_t type, int depth, Value &v) {
        v.type = type;
        switch (type) {
        case 0: { uint8_t x; if (!bytes(&x, 1)) return false; v.u = x; return true; }
        case 1: { int8_t x; if (!bytes(&x, 1)) return false; v.i = x; return true; }
        case 2: { uint16_t x; if (!bytes(&x, 2)) return false; v.u = x; return true; }
        case 3: { int16_t x; if (!bytes(&x, 2)) return false; v.i = x; return true; }
        case 4: { uint32_t x; if (!bytes(&x, 4)) return false; v.u = x; return true; }
        case 5: { int32_t x; if (!bytes(&x, 4)) return false; v.i = x; return true; }
        case 6: { float x; if (!bytes(&x, 4)) return false; v.f = x; return true; }
        case 7: {
            uint8_t x;
            if (!bytes(&x, 1)) return false;
            if (x > 1) return bad(MUMMU_ERR_GGUF, path_ + ": metadata '" + key + "': bool byte " + std::to_string(x));
            v.u = x;
            return true;
        }
        case 8: return string(v.s, "metadata string");
        case 9: {
            if (depth >= 2) return bad(MUMMU_ERR_GGUF, path_ + ": metadata '" + key + "': arrays nested deeper than 2");
            uint32_t elem;
            uint64_t len;
            if (!u32(elem) || !u64(len)) return false;
            if (len > kMaxArrayLen)
                return bad(MUMMU_ERR_GGUF, path_ + ": metadata array of " + std::to_string(len) + " items exceeds the bound " + std::to_string(kMaxArrayLen));
            v.items.resize((size_t)len);
            for (Value &item : v.items)
                if (!value(key, elem, depth + 1, item)) return false;
            return true;
        }
        case 10: return u64(v.u);
        case 11: { int64_t x; if (!bytes(&x, 8)) return false; v.i = x; return true; }
        case 12: { double x; if (!bytes(&x, 8)) return false; v.f = x; return true; }
        default: return bad(MUMMU_ERR_GGUF, path_ + ": metadata '" + key + "': unknown value type " + std::to_string(type));
        }
    }
    long position() { return ftell(f_); }
    bool bad(int c, const std::string &m) {
        code = c;
        err = m;
        return false;
    }

  private:
    static bool valid_utf8(const std::string &s) {
        size_t i = 0;
        const size_t n = s.size();
        while (i < n) {
            const unsigned char c = (unsigned char)s[i];
            size_t extra;
            uint32_t cp;
            if (c < 0x80) { i++; continue; }
            if ((c & 0xE0) == 0xC0) { extra = 1; cp = c & 0x1F; }
            else if ((c & 0xF0) == 0xE0) { extra = 2; cp = c & 0x0F; }
            else if ((c & 0xF8) == 0xF0) { extra = 3; cp = c & 0x07; }
            else return false;
            for (size_t k = 1; k <= extra; k++) {
                if (i + k >= n) return false;
                const unsigned char cc = (unsigned char)s[i + k];
                if ((cc & 0xC0) != 0x80) return false;
                cp = (cp << 6) | (cc & 0x3F);
            }
            if ((extra == 1 && cp < 0x80) || (extra == 2 && cp < 0x800) || (extra == 3 && cp < 0x10000)) return false;  // overlong
            if (cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
            i += extra + 1;
        }
        return true;
    }
    FILE *f_;
    std::string path_;
};

// One file's header.  gguf.rs:1226-1376.
int parse_file(const std::string &path, Parsed &out) {
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return fail(MUMMU_ERR_IO, path + ": cannot open: " + strerror(errno));
    Reader r(f, path);
    auto done = [&](int code, const std::string &msg) {
        fclose(f);
        return code == MUMMU_OK ? MUMMU_OK : fail(code, msg);
    };
    char magic[4];
    if (!r.bytes(magic, 4)) return done(r.code, r.err);
    if (memcmp(magic, "GGUF", 4) != 0) {
        char buf[64];
        snprintf(buf, sizeof(buf), "%02x %02x %02x %02x", (unsigned char)magic[0], (unsigned char)magic[1], (unsigned char)magic[2], (unsigned char)magic[3]);
        return done(MUMMU_ERR_GGUF, path + ": not a GGUF file (magic " + buf + ")");
    }
    uint64_t n_tensors, n_kv;
    if (!r.u32(out.version)) return done(r.code, r.err);
    if (out.version != 2 && out.version != 3) return done(MUMMU_ERR_GGUF, path + ": unsupported GGUF version " + std::to_string(out.version));
    if (!r.u64(n_tensors) || !r.u64(n_kv)) return done(r.code, r.err);
    if (n_tensors > kMaxTensors) return done(MUMMU_ERR_GGUF, path + ": tensor count " + std::to_string(n_tensors) + " exceeds the bound " + std::to_string(kMaxTensors));
    if (n_kv > kMaxKvs) return done(MUMMU_ERR_GGUF, path + ": metadata kv count " + std::to_string(n_kv) + " exceeds the bound " + std::to_string(kMaxKvs));
    out.metadata.reserve((size_t)n_kv);
    for (uint64_t i = 0; i < n_kv; i++) {
        std::string key;
        uint32_t type;
        Value v;
        if (!r.string(key, "metadata key") || !r.u32(type) || !r.value(key, type, 0, v)) return done(r.code, r.err);
        out.metadata.emplace_back(std::move(key), std::move(v));
    }
    out.alignment = kDefaultAlignment;
    for (const auto &kv : out.metadata)
        if (kv.first == "general.alignment") {
            uint64_t a;
            if (kv.second.as_u64(a)) out.alignment = a;
            break;
        }
    if (out.alignment == 0 || (out.alignment & (out.alignment - 1)) != 0)
        return done(MUMMU_ERR_GGUF, path + ": general.alignment " + std::to_string(out.alignment) + " is not a power of two");

    out.tensors.reserve((size_t)n_tensors);
    std::map<std::string, size_t> names;
    for (uint64_t idx = 0; idx < n_tensors; idx++) {
        Tensor t;
        uint32_t n_dims;
        auto bad_tensor = [&](const std::string &why) { return done(MUMMU_ERR_GGUF, path + ": tensor " + std::to_string(idx) + ": " + why); };
        if (!r.string(t.name, "tensor name") || !r.u32(n_dims)) return done(r.code, r.err);
        if (n_dims == 0 || n_dims > kMaxDims) return bad_tensor(std::to_string(n_dims) + " dims (1..=" + std::to_string(kMaxDims) + ")");
        t.dims.resize(n_dims);
        for (uint64_t &d : t.dims)
            if (!r.u64(d)) return done(r.code, r.err);
        if (!r.u32(t.type)) return done(r.code, r.err);
        const TypeInfo *ti = type_info(t.type);
        if (!ti) return bad_tensor("unknown ggml type id " + std::to_string(t.type));
        if (!r.u64(t.offset)) return done(r.code, r.err);
        if (t.offset % out.alignment != 0) return bad_tensor("offset " + std::to_string(t.offset) + " not " + std::to_string(out.alignment) + "-aligned");
        unsigned __int128 elements = 1;
        for (uint64_t d : t.dims) {
            elements *= d;
            if (elements > (unsigned __int128)UINT64_MAX) return bad_tensor("element count overflows");
        }
        const uint64_t el = (uint64_t)elements;
        if (el == 0 || el % ti->block_size != 0) return bad_tensor(std::to_string(el) + " elements is not whole blocks of type " + std::to_string(t.type));
        t.nbytes = el / ti->block_size * ti->block_bytes;
        if (!names.emplace(t.name, (size_t)idx).second) return bad_tensor("duplicate tensor name '" + t.name + "'");
        out.tensors.push_back(std::move(t));
    }
    // payloads must not overlap: a table whose types do not match the file's packing would
    // otherwise hand a neighbour's bytes out as weights
    std::vector<size_t> order(out.tensors.size());
    for (size_t i = 0; i < order.size(); i++) order[i] = i;
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return out.tensors[a].offset < out.tensors[b].offset; });
    for (size_t i = 1; i < order.size(); i++) {
        const Tensor &a = out.tensors[order[i - 1]], &b = out.tensors[order[i]];
        const uint64_t end = a.offset + a.nbytes < a.offset ? UINT64_MAX : a.offset + a.nbytes;
        if (end > b.offset)
            return done(MUMMU_ERR_GGUF, path + ": tensor " + std::to_string(order[i]) + ": '" + b.name + "' at offset " + std::to_string(b.offset) +
                                            " overlaps '" + a.name + "' (" + std::to_string(a.nbytes) + " bytes ending at " + std::to_string(end) + ")");
    }
    const uint64_t header_end = (uint64_t)r.position();
    out.data_offset = (header_end + out.alignment - 1) / out.alignment * out.alignment;
    return done(MUMMU_OK, "");
}

const Value *find_value(const Parsed &p, const std::string &key) {
    for (const auto &kv : p.metadata)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

bool is_file(const std::string &p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

// Every shard path of a split set from one member's name `<stem>-NNNNN-of-NNNNN.gguf`.
int shard_paths(const std::string &member, uint64_t count, std::vector<std::string> &out) {
    const size_t slash = member.find_last_of('/');
    const std::string dir = slash == std::string::npos ? "" : member.substr(0, slash + 1);
    const std::string name = slash == std::string::npos ? member : member.substr(slash + 1);
    auto bad = [&](const std::string &why) { return fail(MUMMU_ERR_GGUF, member + ": split filename: " + why); };
    if (name.size() < 5 || name.compare(name.size() - 5, 5, ".gguf") != 0) return bad("shard filename does not end in .gguf");
    const std::string stem = name.substr(0, name.size() - 5);
    const size_t of = stem.rfind("-of-");  // from the right: a model name may contain "-of-" itself
    if (of == std::string::npos) return bad(name + ": split.count > 1 but the name has no -of- index");
    const std::string head = stem.substr(0, of);
    const size_t dash = head.rfind('-');
    if (dash == std::string::npos) return bad(name + ": no -NNNNN- shard index before -of-");
    const std::string base = head.substr(0, dash);
    for (uint64_t i = 1; i <= count; i++) {
        char buf[48];
        snprintf(buf, sizeof(buf), "-%05llu-of-%05llu.gguf", (unsigned long long)i, (unsigned long long)count);
        out.push_back(dir + base + buf);
    }
    for (const std::string &p : out)
        if (!is_file(p)) return bad("missing shard " + p);
    return MUMMU_OK;
}

}  // namespace

struct mummu_gguf {
    Parsed header;              // version, alignment, metadata of the shard that carries it; merged tensor table
    std::vector<Shard> shards;  // one per file (one entry for a single-file GGUF)
    std::string arch;
    ~mummu_gguf() {
        for (Shard &s : shards) {
            if (s.map) munmap(s.map, s.map_len);
            if (s.fd >= 0) close(s.fd);
        }
    }
    int find(const std::string &name) const {
        for (size_t i = 0; i < header.tensors.size(); i++)
            if (header.tensors[i].name == name) return (int)i;
        return -1;
    }
    // Maps the shard's file on first use; returns the payload bytes of a tensor.
    int payload(int index, const void **data) {
        const Tensor &t = header.tensors[(size_t)index];
        Shard &s = shards[(size_t)t.shard];
        if (!s.map) {
            s.fd = open(s.path.c_str(), O_RDONLY);
            if (s.fd < 0) return fail(MUMMU_ERR_IO, s.path + ": cannot open: " + strerror(errno));
            struct stat st;
            if (fstat(s.fd, &st) != 0) return fail(MUMMU_ERR_IO, s.path + ": cannot stat");
            s.map_len = (size_t)st.st_size;
            s.map = mmap(nullptr, s.map_len, PROT_READ, MAP_PRIVATE, s.fd, 0);
            if (s.map == MAP_FAILED) {
                s.map = nullptr;
                return fail(MUMMU_ERR_IO, s.path + ": cannot map");
            }
        }
        const uint64_t begin = s.data_offset + t.offset;
        if (begin + t.nbytes < begin || begin + t.nbytes > s.map_len)
            return fail(MUMMU_ERR_GGUF, s.path + ": tensor '" + t.name + "' (" + std::to_string(t.nbytes) + " bytes at " + std::to_string(begin) +
                                            ") runs past the end of the file (" + std::to_string(s.map_len) + " bytes)");
        *data = (const uint8_t *)s.map + begin;
        return MUMMU_OK;
    }
};

extern "C" {

const char *mummu_gguf_last_error(void) { return g_gguf_error.c_str(); }

int mummu_gguf_open(const char *path, mummu_gguf **out) {
    if (!path || !out) return fail(MUMMU_ERR_ARG, "null path or output pointer");
    *out = nullptr;
    Parsed first;
    int rc = parse_file(path, first);
    if (rc) return rc;
    mummu_gguf *g = new mummu_gguf();
    auto bail = [&](int code) {
        delete g;
        return code;
    };
    uint64_t count = 0;
    const Value *sc = find_value(first, "split.count");
    if (!sc || !sc->as_u64(count) || count <= 1) {
        Shard s;
        s.path = path;
        s.data_offset = first.data_offset;
        g->shards.push_back(s);
        g->header = std::move(first);
    } else {
        if (count > kMaxShards) return bail(fail(MUMMU_ERR_GGUF, std::string(path) + ": split.count: " + std::to_string(count) + " shards exceeds the " + std::to_string(kMaxShards) + " bound"));
        std::vector<std::string> paths;
        if ((rc = shard_paths(path, count, paths))) return bail(rc);
        std::vector<Tensor> tensors;
        size_t best_kv = 0;
        bool have = false;
        for (size_t si = 0; si < paths.size(); si++) {
            Parsed p;
            if ((rc = parse_file(paths[si], p))) return bail(rc);
            Shard s;
            s.path = paths[si];
            s.data_offset = p.data_offset;
            g->shards.push_back(s);
            for (Tensor &t : p.tensors) {
                t.shard = (int)si;
                tensors.push_back(std::move(t));
            }
            p.tensors.clear();
            if (!have || p.metadata.size() > best_kv) {  // the richest key-value set is the real metadata
                best_kv = p.metadata.size();
                g->header = std::move(p);
                have = true;
            }
        }
        std::map<std::string, int> seen;
        for (const Tensor &t : tensors)
            if (!seen.emplace(t.name, 1).second)
                return bail(fail(MUMMU_ERR_GGUF, std::string(path) + ": " + t.name + ": tensor name appears in more than one shard"));
        const Value *declared = find_value(first, "split.tensors.count");
        uint64_t want;
        if (declared && declared->as_u64(want) && want != tensors.size())
            return bail(fail(MUMMU_ERR_GGUF, std::string(path) + ": split.tensors.count: header declares " + std::to_string(want) + " tensors, shards carry " + std::to_string(tensors.size())));
        g->header.tensors = std::move(tensors);
    }
    const Value *arch = find_value(g->header, "general.architecture");
    if (arch && arch->type == 8) g->arch = arch->s;
    *out = g;
    return MUMMU_OK;
}

void mummu_gguf_close(mummu_gguf *g) { delete g; }

int mummu_gguf_version(const mummu_gguf *g) { return g ? (int)g->header.version : -1; }
int64_t mummu_gguf_alignment(const mummu_gguf *g) { return g ? (int64_t)g->header.alignment : -1; }
int mummu_gguf_shard_count(const mummu_gguf *g) { return g ? (int)g->shards.size() : -1; }
int mummu_gguf_tensor_count(const mummu_gguf *g) { return g ? (int)g->header.tensors.size() : -1; }
int mummu_gguf_kv_count(const mummu_gguf *g) { return g ? (int)g->header.metadata.size() : -1; }
int mummu_gguf_find_tensor(const mummu_gguf *g, const char *name) { return (g && name) ? g->find(name) : -1; }

int mummu_gguf_tensor_info(const mummu_gguf *g, int index, mummu_gguf_tensor *out) {
    if (!g || !out) return fail(MUMMU_ERR_ARG, "null argument");
    if (index < 0 || index >= (int)g->header.tensors.size()) return fail(MUMMU_ERR_RANGE, "tensor index " + std::to_string(index) + " out of range");
    const Tensor &t = g->header.tensors[(size_t)index];
    const Shard &s = g->shards[(size_t)t.shard];
    out->name = t.name.c_str();
    out->n_dims = (int32_t)t.dims.size();
    for (int i = 0; i < 4; i++) out->dims[i] = i < (int)t.dims.size() ? (int64_t)t.dims[(size_t)i] : 1;
    out->ggml_type = (int32_t)t.type;
    out->shard = t.shard;
    out->file_offset = s.data_offset + t.offset;
    out->nbytes = t.nbytes;
    out->path = s.path.c_str();
    return MUMMU_OK;
}

int mummu_gguf_tensor_data(mummu_gguf *g, int index, const void **data, uint64_t *nbytes) {
    if (!g || !data) return fail(MUMMU_ERR_ARG, "null argument");
    if (index < 0 || index >= (int)g->header.tensors.size()) return fail(MUMMU_ERR_RANGE, "tensor index " + std::to_string(index) + " out of range");
    if (nbytes) *nbytes = g->header.tensors[(size_t)index].nbytes;
    return g->payload(index, data);
}

int mummu_gguf_get_u64(const mummu_gguf *g, const char *key, uint64_t *out) {
    if (!g || !key || !out) return fail(MUMMU_ERR_ARG, "null argument");
    const Value *v = find_value(g->header, key);
    if (!v) return fail(MUMMU_ERR_NOT_LOADED, std::string("GGUF has no metadata key ") + key);
    if (v->type == 7) {  // as_bool (gguf.rs:183-188) shares this getter: 0 or 1
        *out = v->u;
        return MUMMU_OK;
    }
    if (!v->as_u64(*out)) return fail(MUMMU_ERR_TYPE, std::string("GGUF metadata ") + key + " is not an unsigned integer");
    return MUMMU_OK;
}

int mummu_gguf_get_f64(const mummu_gguf *g, const char *key, double *out) {
    if (!g || !key || !out) return fail(MUMMU_ERR_ARG, "null argument");
    const Value *v = find_value(g->header, key);
    if (!v) return fail(MUMMU_ERR_NOT_LOADED, std::string("GGUF has no metadata key ") + key);
    if (v->type != 6 && v->type != 12) return fail(MUMMU_ERR_TYPE, std::string("GGUF metadata ") + key + " is not a float");
    *out = v->f;
    return MUMMU_OK;
}

const char *mummu_gguf_get_str(const mummu_gguf *g, const char *key) {
    if (!g || !key) return nullptr;
    const Value *v = find_value(g->header, key);
    return (v && v->type == 8) ? v->s.c_str() : nullptr;
}

// The MoE block's configuration from the header (models/olmoe.rs:116-179): keys live under the
// architecture's prefix; the per-expert width is expert_feed_forward_length when present.
int mummu_gguf_moe_config(const mummu_gguf *g, mummu_moe_config *cfg) {
    if (!g || !cfg) return fail(MUMMU_ERR_ARG, "null argument");
    if (g->arch.empty()) return fail(MUMMU_ERR_GGUF, "GGUF has no general.architecture");
    const std::string a = g->arch + ".";
    auto need = [&](const std::string &key, uint64_t &v) {
        const Value *val = find_value(g->header, a + key);
        if (!val || !val->as_u64(v)) return fail(MUMMU_ERR_GGUF, "GGUF metadata " + a + key + " is missing or not an unsigned integer");
        return (int)MUMMU_OK;
    };
    uint64_t hidden, inter, experts, used, layers;
    int rc;
    if ((rc = need("embedding_length", hidden))) return rc;
    if (need("expert_feed_forward_length", inter) != MUMMU_OK && (rc = need("feed_forward_length", inter))) return rc;
    if ((rc = need("expert_count", experts)) || (rc = need("expert_used_count", used)) || (rc = need("block_count", layers))) return rc;
    const uint64_t lim = 1u << 30;
    if (hidden > lim || inter > lim || experts > lim || used > lim || layers > lim) return fail(MUMMU_ERR_GGUF, "GGUF MoE dimensions are out of range");
    memset(cfg, 0, sizeof(*cfg));
    cfg->hidden_size = (int32_t)hidden;
    cfg->expert_intermediate_size = (int32_t)inter;
    cfg->num_experts = (int32_t)experts;
    cfg->num_experts_per_tok = (int32_t)used;
    cfg->num_layers = (int32_t)layers;
    const Value *norm = find_value(g->header, a + "expert_weights_norm");
    cfg->norm_topk_prob = (norm && norm->type == 7) ? (int32_t)norm->u : 0;
    const Value *eps = find_value(g->header, a + "attention.layer_norm_rms_epsilon");
    if (!eps || eps->type != 6) return fail(MUMMU_ERR_GGUF, "GGUF metadata " + a + "attention.layer_norm_rms_epsilon is missing or not an f32");
    cfg->rms_norm_eps = (float)eps->f;
    cfg->router_flavour = MUMMU_ROUTER_SPARSE_MOE;
    cfg->max_tokens = 512;
    // models/olmoe.rs:210-215, nn/moe.rs:62-76
    if (cfg->num_experts < 2) return fail(MUMMU_ERR_CONFIG, "GGUF header: num_experts must be >= 2 (got " + std::to_string(cfg->num_experts) + ")");
    if (cfg->num_experts_per_tok < 1 || cfg->num_experts_per_tok > cfg->num_experts)
        return fail(MUMMU_ERR_CONFIG, "GGUF header: num_experts_per_tok (" + std::to_string(cfg->num_experts_per_tok) + ") must be in 1..=num_experts (" + std::to_string(cfg->num_experts) + ")");
    g_gguf_error.clear();
    return MUMMU_OK;
}

// The expert-bank locator for one layer: the five tensors by name, their dims checked against
// the header's configuration (GGUF order, fastest first: router [H,E], gate/up [H,I,E], down
// [I,H,E], norm [H]) and each bank row checked to be whole blocks.
int mummu_gguf_locate_moe_layer(const mummu_gguf *g, int layer, mummu_gguf_moe_layer *out) {
    if (!g || !out) return fail(MUMMU_ERR_ARG, "null argument");
    mummu_moe_config want;
    int rc = mummu_gguf_moe_config(g, &want);
    if (rc) return rc;
    if (layer < 0 || layer >= want.num_layers)
        return fail(MUMMU_ERR_RANGE, "layer " + std::to_string(layer) + " is not inside the file's " + std::to_string(want.num_layers) + " blocks");
    const std::string blk = "blk." + std::to_string(layer) + ".";
    auto locate = [&](const std::string &suffix, int n_dims, const uint64_t *dims, int32_t &index, bool optional) {
        const std::string name = blk + suffix;
        index = g->find(name);
        if (index < 0) return optional ? (int)MUMMU_OK : fail(MUMMU_ERR_GGUF, "GGUF has no " + name);
        const Tensor &t = g->header.tensors[(size_t)index];
        if ((int)t.dims.size() != n_dims) return fail(MUMMU_ERR_SHAPE, name + " has " + std::to_string(t.dims.size()) + " dims, want " + std::to_string(n_dims));
        for (int i = 0; i < n_dims; i++)
            if (t.dims[(size_t)i] != dims[i])
                return fail(MUMMU_ERR_SHAPE, name + ": dim " + std::to_string(i) + " is " + std::to_string(t.dims[(size_t)i]) + ", the header's configuration wants " + std::to_string(dims[i]));
        const TypeInfo *ti = type_info(t.type);
        // whole blocks per ROW, not only per tensor (experts.rs:150-154)
        if (dims[0] % ti->block_size != 0)
            return fail(MUMMU_ERR_BLOCKS, name + ": a row of " + std::to_string(dims[0]) + " elements is not whole blocks of type " + std::to_string(t.type));
        // experts.rs:900-904: the geometry must account for every byte the header gives the tensor
        uint64_t rows = 1;
        for (int i = 1; i < n_dims; i++) rows *= dims[i];
        if (rows * (dims[0] / ti->block_size) * ti->block_bytes != t.nbytes)
            return fail(MUMMU_ERR_SHAPE, name + ": bank geometry disagrees with the header's byte length");
        return (int)MUMMU_OK;
    };
    const uint64_t H = (uint64_t)want.hidden_size, I = (uint64_t)want.expert_intermediate_size, E = (uint64_t)want.num_experts;
    const uint64_t d_router[2] = {H, E}, d_fwd[3] = {H, I, E}, d_back[3] = {I, H, E}, d_norm[1] = {H};
    if ((rc = locate("ffn_gate_inp.weight", 2, d_router, out->router, false)) || (rc = locate("ffn_gate_exps.weight", 3, d_fwd, out->gate, false)) ||
        (rc = locate("ffn_up_exps.weight", 3, d_fwd, out->up, false)) || (rc = locate("ffn_down_exps.weight", 3, d_back, out->down, false)) ||
        (rc = locate("ffn_norm.weight", 1, d_norm, out->norm, true)))
        return rc;
    if (out->norm >= 0 && g->header.tensors[(size_t)out->norm].type != MUMMU_F32) return fail(MUMMU_ERR_TYPE, blk + "ffn_norm.weight must be F32");
    g_gguf_error.clear();
    return MUMMU_OK;
}

// Locate and load the MoE block of layers [first_layer, first_layer + n_layers) into the
// handle's layers 0.. : router, the three fused banks and the pre-norm weight, bytes unchanged.
int mummu_moe_load_gguf(mummu_moe *h, mummu_gguf *g, int first_layer, int n_layers) {
    if (!h || !g) return fail(MUMMU_ERR_ARG, "null argument");
    if (first_layer < 0 || n_layers < 1) return fail(MUMMU_ERR_RANGE, "first_layer must be >= 0 and n_layers >= 1");
    {
        // the handle reads its banks by its own geometry: a file of another geometry would be read past its tensors
        mummu_moe_config have, file;
        int rc = mummu_moe_get_config(h, &have);
        if (rc) return fail(rc, "the handle's configuration could not be read");
        if ((rc = mummu_gguf_moe_config(g, &file))) return rc;
        if (have.hidden_size != file.hidden_size || have.expert_intermediate_size != file.expert_intermediate_size ||
            have.num_experts != file.num_experts)
            return fail(MUMMU_ERR_SHAPE, "the handle was created for hidden " + std::to_string(have.hidden_size) + ", intermediate " +
                                             std::to_string(have.expert_intermediate_size) + ", " + std::to_string(have.num_experts) +
                                             " experts; the file holds hidden " + std::to_string(file.hidden_size) + ", intermediate " +
                                             std::to_string(file.expert_intermediate_size) + ", " + std::to_string(file.num_experts) + " experts");
        if (n_layers > have.num_layers)
            return fail(MUMMU_ERR_RANGE, std::to_string(n_layers) + " layers do not fit the handle's " + std::to_string(have.num_layers));
    }
    for (int l = 0; l < n_layers; l++) {
        mummu_gguf_moe_layer at;
        int rc = mummu_gguf_locate_moe_layer(g, first_layer + l, &at);
        if (rc) return rc;
        const int32_t index[5] = {at.router, at.gate, at.up, at.down, at.norm};
        const void *data[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
        int type[5] = {0, 0, 0, 0, 0};
        for (int i = 0; i < 5; i++) {
            if (index[i] < 0) continue;
            type[i] = (int)g->header.tensors[(size_t)index[i]].type;
            if ((rc = g->payload(index[i], &data[i]))) return rc;
        }
        rc = mummu_moe_load_layer(h, l, data[0], type[0], data[1], type[1], data[2], type[2], data[3], type[3], (const float *)data[4]);
        if (rc) return fail(rc, "blk." + std::to_string(first_layer + l) + ": " + mummu_moe_last_error(h));
        // the shared expert of a Qwen-style block, when the file has one (models/qwen4exp/model.rs:228-231)
        const std::string blk = "blk." + std::to_string(first_layer + l) + ".";
        const int sg = g->find(blk + "ffn_gate_shexp.weight"), su = g->find(blk + "ffn_up_shexp.weight"),
                  sd = g->find(blk + "ffn_down_shexp.weight"), sv = g->find(blk + "ffn_gate_inp_shexp.weight");
        if (sg >= 0 || su >= 0 || sd >= 0) {
            if (sg < 0 || su < 0 || sd < 0) return fail(MUMMU_ERR_GGUF, blk + "ffn_*_shexp.weight: the shared expert needs its gate, up and down tensors");
            const Tensor &tg = g->header.tensors[(size_t)sg], &tu = g->header.tensors[(size_t)su], &td = g->header.tensors[(size_t)sd];
            mummu_moe_config want;
            if ((rc = mummu_gguf_moe_config(g, &want))) return rc;
            const uint64_t H = (uint64_t)want.hidden_size;
            if (tg.dims.size() != 2 || tu.dims.size() != 2 || td.dims.size() != 2 || tg.dims[0] != H || tu.dims != tg.dims ||
                td.dims[0] != tg.dims[1] || td.dims[1] != H || tg.dims[1] > (1u << 30))
                return fail(MUMMU_ERR_SHAPE, blk + "ffn_*_shexp.weight: want gate/up [hidden, width] and down [width, hidden]");
            const void *pg, *pu, *pd, *pv = nullptr;
            int vt = MUMMU_F32;
            if ((rc = g->payload(sg, &pg)) || (rc = g->payload(su, &pu)) || (rc = g->payload(sd, &pd))) return rc;
            if (sv >= 0) {
                const Tensor &tv = g->header.tensors[(size_t)sv];
                if (tv.dims.size() != 1 || tv.dims[0] != H) return fail(MUMMU_ERR_SHAPE, blk + "ffn_gate_inp_shexp.weight: want [hidden]");
                vt = (int)tv.type;
                if ((rc = g->payload(sv, &pv))) return rc;
            }
            rc = mummu_moe_load_shared_expert(h, l, (int)tg.dims[1], pg, (int)tg.type, pu, (int)tu.type, pd, (int)td.type, pv, vt);
            if (rc) return fail(rc, blk + "ffn_*_shexp: " + mummu_moe_last_error(h));
        }
    }
    g_gguf_error.clear();
    return MUMMU_OK;
}

}  // extern "C"
