// HF safetensors checkpoint directories for the MoE block (host only): `config.json` parsing
// and validation, shard discovery, header parsing with every entry checked against the payload
// it claims, and the expert fuse - `model.layers.L.mlp.experts.I.{gate,up,down}_proj.weight`
// ([out, in] each) stacked in numeric expert order into the `[E, out, in]` banks the kernels
// read, source dtype (BF16 / F16 / F32) preserved.
//
// Reference behaviour followed (physics515/Mummu, crates/mummu/src/): models/olmoe.rs:52-226
// (OlmoeConfig fields, defaults and validation), :405-430 (which names fuse where);
// safetensors.rs:39-58 (bounds), :180-320 (header rules), :332-341 (dtype sizes), :377-430
// (shards), :600-740 (group rules: index range, count agreement, duplicates, completeness,
// layout agreement, numeric member order).
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/mummu_moe.h"

namespace {

constexpr uint64_t kMaxHeaderBytes = 64ull << 20, kMaxTensors = 1ull << 20, kMaxShards = 256, kMaxPartBytes = 4ull << 30;

thread_local std::string g_st_error;

int fail(int code, const std::string &msg) {
    g_st_error = msg;
    return code;
}

// ---- a small JSON reader (RFC 8259 values; numbers keep whether they were plain integers) -------
struct Json {
    enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
    bool b = false;
    double num = 0.0;
    bool is_uint = false;  // a non-negative integer literal without fraction or exponent that fits u64
    uint64_t u = 0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;  // file order

    const Json *get(const std::string &key) const {
        if (kind != Obj) return nullptr;
        for (const auto &kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
};

class JsonParser {
  public:
    JsonParser(const char *p, size_t n) : p_(p), end_(p + n) {}
    bool parse(Json &out, std::string &err) {
        if (!value(out, 0) || (ws(), p_ != end_)) {
            if (err_.empty()) err_ = "trailing characters after the JSON value";
            err = err_ + " at byte " + std::to_string((size_t)(p_ - start()));
            return false;
        }
        return true;
    }

  private:
    const char *start() const { return end_ - total_; }
    void ws() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) p_++;
    }
    bool bad(const char *why) {
        if (err_.empty()) err_ = why;
        return false;
    }
    bool literal(const char *word) {
        const size_t n = strlen(word);
        if ((size_t)(end_ - p_) < n || memcmp(p_, word, n) != 0) return bad("unknown literal");
        p_ += n;
        return true;
    }
    static void utf8(std::string &s, uint32_t cp) {
        if (cp < 0x80) s += (char)cp;
        else if (cp < 0x800) { s += (char)(0xC0 | (cp >> 6)); s += (char)(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) { s += (char)(0xE0 | (cp >> 12)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F)); }
        else { s += (char)(0xF0 | (cp >> 18)); s += (char)(0x80 | ((cp >> 12) & 0x3F)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F)); }
    }
    bool hex4(uint32_t &v) {
        if (end_ - p_ < 4) return bad("short \\u escape");
        v = 0;
        for (int i = 0; i < 4; i++) {
            const char c = *p_++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
            else return bad("bad \\u escape");
        }
        return true;
    }
    bool string(std::string &s) {
        p_++;  // opening quote
        while (p_ < end_) {
            const unsigned char c = (unsigned char)*p_++;
            if (c == '"') return true;
            if (c < 0x20) return bad("control character in a string");
            if (c != '\\') {
                s += (char)c;
                continue;
            }
            if (p_ >= end_) break;
            const char e = *p_++;
            switch (e) {
            case '"': s += '"'; break;
            case '\\': s += '\\'; break;
            case '/': s += '/'; break;
            case 'b': s += '\b'; break;
            case 'f': s += '\f'; break;
            case 'n': s += '\n'; break;
            case 'r': s += '\r'; break;
            case 't': s += '\t'; break;
            case 'u': {
                uint32_t cp;
                if (!hex4(cp)) return false;
                if (cp >= 0xD800 && cp < 0xDC00) {  // surrogate pair
                    uint32_t lo;
                    if (end_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') return bad("lone surrogate");
                    p_ += 2;
                    if (!hex4(lo) || lo < 0xDC00 || lo > 0xDFFF) return bad("lone surrogate");
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
                    return bad("lone surrogate");
                }
                utf8(s, cp);
                break;
            }
            default: return bad("bad escape");
            }
        }
        return bad("unterminated string");
    }
    bool number(Json &out) {
        const char *s = p_;
        if (p_ < end_ && *p_ == '-') p_++;
        if (p_ >= end_ || *p_ < '0' || *p_ > '9') return bad("bad number");
        if (*p_ == '0') p_++;
        else while (p_ < end_ && *p_ >= '0' && *p_ <= '9') p_++;
        bool plain = true;
        if (p_ < end_ && *p_ == '.') {
            plain = false;
            p_++;
            if (p_ >= end_ || *p_ < '0' || *p_ > '9') return bad("bad number");
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') p_++;
        }
        if (p_ < end_ && (*p_ == 'e' || *p_ == 'E')) {
            plain = false;
            p_++;
            if (p_ < end_ && (*p_ == '+' || *p_ == '-')) p_++;
            if (p_ >= end_ || *p_ < '0' || *p_ > '9') return bad("bad number");
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') p_++;
        }
        const std::string tok(s, (size_t)(p_ - s));
        out.kind = Json::Num;
        out.num = strtod(tok.c_str(), nullptr);
        if (plain && tok[0] != '-') {
            unsigned __int128 v = 0;
            bool fits = true;
            for (char c : tok) {
                v = v * 10 + (unsigned)(c - '0');
                if (v > (unsigned __int128)UINT64_MAX) {
                    fits = false;
                    break;
                }
            }
            out.is_uint = fits;
            out.u = fits ? (uint64_t)v : 0;
        }
        return true;
    }
    bool value(Json &out, int depth) {
        if (depth > 64) return bad("nested too deep");
        ws();
        if (p_ >= end_) return bad("unexpected end");
        switch (*p_) {
        case '{': {
            out.kind = Json::Obj;
            p_++;
            ws();
            if (p_ < end_ && *p_ == '}') { p_++; return true; }
            for (;;) {
                ws();
                if (p_ >= end_ || *p_ != '"') return bad("object key must be a string");
                std::string key;
                if (!string(key)) return false;
                ws();
                if (p_ >= end_ || *p_ != ':') return bad("missing ':'");
                p_++;
                Json v;
                if (!value(v, depth + 1)) return false;
                out.obj.emplace_back(std::move(key), std::move(v));
                ws();
                if (p_ < end_ && *p_ == ',') { p_++; continue; }
                if (p_ < end_ && *p_ == '}') { p_++; return true; }
                return bad("missing ',' or '}'");
            }
        }
        case '[': {
            out.kind = Json::Arr;
            p_++;
            ws();
            if (p_ < end_ && *p_ == ']') { p_++; return true; }
            for (;;) {
                Json v;
                if (!value(v, depth + 1)) return false;
                out.arr.push_back(std::move(v));
                ws();
                if (p_ < end_ && *p_ == ',') { p_++; continue; }
                if (p_ < end_ && *p_ == ']') { p_++; return true; }
                return bad("missing ',' or ']'");
            }
        }
        case '"': out.kind = Json::Str; return string(out.str);
        case 't': out.kind = Json::Bool; out.b = true; return literal("true");
        case 'f': out.kind = Json::Bool; out.b = false; return literal("false");
        case 'n': out.kind = Json::Null; return literal("null");
        default: return number(out);
        }
    }
    const char *p_, *end_;
    size_t total_ = (size_t)(end_ - p_);
    std::string err_;
};

bool read_file(const std::string &path, std::string &out, std::string &err) {
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) {
        err = path + ": cannot open: " + strerror(errno);
        return false;
    }
    char buf[1 << 16];
    size_t n;
    while ((n = fread(buf, 1, sizeof(buf), f)) > 0) out.append(buf, n);
    fclose(f);
    return true;
}

bool is_file(const std::string &p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

// safetensors.rs:332-341
int dtype_bytes(const std::string &d) {
    if (d == "BOOL" || d == "U8" || d == "I8" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
    if (d == "U16" || d == "I16" || d == "F16" || d == "BF16") return 2;
    if (d == "U32" || d == "I32" || d == "F32") return 4;
    if (d == "U64" || d == "I64" || d == "F64") return 8;
    return 0;
}

struct Entry {
    std::string name, dtype;
    std::vector<uint64_t> shape;
    uint64_t start = 0, end = 0;  // inside the shard's payload
    int shard = 0;
};

struct ShardFile {
    std::string path;
    uint64_t data_offset = 0;
    int fd = -1;
};

// One shard's header (safetensors.rs:180-320).
int parse_shard(const std::string &path, int shard, ShardFile &sf, std::vector<Entry> &out) {
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return fail(MUMMU_ERR_IO, path + ": cannot open: " + strerror(errno));
    struct stat st;
    if (fstat(fileno(f), &st) != 0) {
        fclose(f);
        return fail(MUMMU_ERR_IO, path + ": cannot stat");
    }
    const uint64_t file_len = (uint64_t)st.st_size;
    uint64_t header_len = 0;
    if (fread(&header_len, 1, 8, f) != 8) {
        fclose(f);
        return fail(MUMMU_ERR_IO, path + ": file ends inside the header length");
    }
    if (header_len > kMaxHeaderBytes || header_len + 8 > file_len) {
        fclose(f);
        return fail(MUMMU_ERR_SAFETENSORS, path + ": header bytes " + std::to_string(header_len) + " exceeds the bound " +
                                               std::to_string(std::min(kMaxHeaderBytes, file_len)));
    }
    std::string header((size_t)header_len, '\0');
    const bool ok = fread(&header[0], 1, (size_t)header_len, f) == (size_t)header_len;
    fclose(f);
    if (!ok) return fail(MUMMU_ERR_IO, path + ": file ends inside the header");
    sf.path = path;
    sf.data_offset = 8 + header_len;
    const uint64_t payload_len = file_len - sf.data_offset;

    Json json;
    std::string err;
    if (!JsonParser(header.data(), header.size()).parse(json, err)) return fail(MUMMU_ERR_SAFETENSORS, path + ": bad header: " + err);
    if (json.kind != Json::Obj) return fail(MUMMU_ERR_SAFETENSORS, path + ": bad header: header is not a JSON object");
    if (json.obj.size() > kMaxTensors)
        return fail(MUMMU_ERR_SAFETENSORS, path + ": tensor entries " + std::to_string(json.obj.size()) + " exceeds the bound " + std::to_string(kMaxTensors));
    for (const auto &kv : json.obj) {
        if (kv.first == "__metadata__") continue;  // a free-form string map, not a tensor
        auto bad = [&](const std::string &why) { return fail(MUMMU_ERR_SAFETENSORS, path + ": tensor '" + kv.first + "': " + why); };
        const Json &e = kv.second;
        if (e.kind != Json::Obj) return bad("entry is not an object");
        Entry t;
        t.name = kv.first;
        t.shard = shard;
        const Json *dt = e.get("dtype");
        if (!dt || dt->kind != Json::Str) return bad("missing 'dtype'");
        t.dtype = dt->str;
        const int eb = dtype_bytes(t.dtype);
        if (!eb) return bad("unsupported dtype '" + t.dtype + "'");
        const Json *shape = e.get("shape");
        if (!shape || shape->kind != Json::Arr) return bad("missing 'shape'");
        for (const Json &d : shape->arr) {
            if (d.kind != Json::Num || !d.is_uint) return bad("non-integer dim");
            t.shape.push_back(d.u);
        }
        const Json *off = e.get("data_offsets");
        if (!off || off->kind != Json::Arr) return bad("missing 'data_offsets'");
        if (off->arr.size() != 2) return bad("data_offsets has " + std::to_string(off->arr.size()) + " entries");
        if (off->arr[0].kind != Json::Num || !off->arr[0].is_uint || off->arr[1].kind != Json::Num || !off->arr[1].is_uint)
            return bad("non-integer data_offset");
        t.start = off->arr[0].u;
        t.end = off->arr[1].u;
        if (t.end < t.start || t.end > payload_len)
            return bad("data_offsets [" + std::to_string(t.start) + ", " + std::to_string(t.end) + ") outside the " + std::to_string(payload_len) + "-byte payload");
        unsigned __int128 expected = (unsigned)eb;
        for (uint64_t d : t.shape) {
            expected *= d;
            if (expected > (unsigned __int128)UINT64_MAX) return bad("shape overflows u64 bytes");
        }
        if ((uint64_t)expected != t.end - t.start)
            return bad("shape of " + t.dtype + " implies " + std::to_string((uint64_t)expected) + " bytes, header claims " + std::to_string(t.end - t.start));
        out.push_back(std::move(t));
    }
    return MUMMU_OK;
}

int ggml_type_of(const std::string &dtype) {
    if (dtype == "F32") return MUMMU_F32;
    if (dtype == "F16") return MUMMU_F16;
    if (dtype == "BF16") return MUMMU_BF16;
    return -1;
}

// The MoE fields of an HF config.json (models/olmoe.rs:52-88) and the checks on them (:180-226).
int config_from_json(const Json &j, const std::string &whose, mummu_moe_config *cfg) {
    if (j.kind != Json::Obj) return fail(MUMMU_ERR_CONFIG, whose + ": config is not a JSON object");
    auto need = [&](const char *key, uint64_t &v) {
        const Json *x = j.get(key);
        if (!x) return fail(MUMMU_ERR_CONFIG, whose + ": missing field `" + key + "`");
        if (x->kind != Json::Num || !x->is_uint) return fail(MUMMU_ERR_CONFIG, whose + ": `" + key + "` is not an unsigned integer");
        v = x->u;
        return (int)MUMMU_OK;
    };
    uint64_t vocab, hidden, inter, layers, heads, kv_heads, experts, used;
    int rc;
    if ((rc = need("vocab_size", vocab)) || (rc = need("hidden_size", hidden)) || (rc = need("intermediate_size", inter)) ||
        (rc = need("num_hidden_layers", layers)) || (rc = need("num_attention_heads", heads)) ||
        (rc = need("num_key_value_heads", kv_heads)) || (rc = need("num_experts", experts)) ||
        (rc = need("num_experts_per_tok", used)))
        return rc;
    const Json *eps = j.get("rms_norm_eps");
    if (!eps || eps->kind != Json::Num) return fail(MUMMU_ERR_CONFIG, whose + ": missing field `rms_norm_eps`");
    bool norm = false;
    if (const Json *n = j.get("norm_topk_prob")) {
        if (n->kind != Json::Bool) return fail(MUMMU_ERR_CONFIG, whose + ": `norm_topk_prob` is not a bool");
        norm = n->b;
    }
    // models/olmoe.rs:195-224, the checks that need only these fields (rope scaling and sliding
    // windows are the attention side's to refuse)
    if (kv_heads == 0 || heads % kv_heads != 0)
        return fail(MUMMU_ERR_CONFIG, whose + ": num_attention_heads (" + std::to_string(heads) + ") must be a positive multiple of num_key_value_heads (" + std::to_string(kv_heads) + ")");
    if (layers == 0 || vocab == 0) return fail(MUMMU_ERR_CONFIG, whose + ": num_hidden_layers and vocab_size must be positive");
    if (experts < 2 || used < 1 || used > experts)
        return fail(MUMMU_ERR_CONFIG, whose + ": num_experts (" + std::to_string(experts) + ") must be >= 2 with num_experts_per_tok (" + std::to_string(used) + ") in 1..=num_experts");
    const uint64_t hd = hidden / std::max<uint64_t>(heads, 1);
    if (hd < 2 || hd % 2 != 0 || hd * heads != hidden)
        return fail(MUMMU_ERR_CONFIG, whose + ": hidden_size (" + std::to_string(hidden) + ") must split evenly into num_attention_heads (" + std::to_string(heads) + ") even-sized heads");
    const uint64_t lim = 1u << 30;
    if (hidden > lim || inter > lim || inter == 0 || experts > lim || layers > lim) return fail(MUMMU_ERR_CONFIG, whose + ": dimensions out of range");
    memset(cfg, 0, sizeof(*cfg));
    cfg->hidden_size = (int32_t)hidden;
    cfg->expert_intermediate_size = (int32_t)inter;
    cfg->num_experts = (int32_t)experts;
    cfg->num_experts_per_tok = (int32_t)used;
    cfg->norm_topk_prob = norm ? 1 : 0;
    cfg->router_flavour = MUMMU_ROUTER_SPARSE_MOE;
    cfg->num_layers = (int32_t)layers;
    cfg->max_tokens = 512;
    cfg->rms_norm_eps = (float)eps->num;
    return MUMMU_OK;
}

}  // namespace

struct mummu_st {
    std::string dir;
    std::vector<ShardFile> shards;
    std::vector<Entry> tensors;  // every shard's entries, each shard's in payload order
    std::map<std::string, int> by_name;
    mummu_moe_config cfg{};
    bool have_cfg = false;
    std::string cfg_error;
    int cfg_status = MUMMU_OK;
    ~mummu_st() {
        for (ShardFile &s : shards)
            if (s.fd >= 0) close(s.fd);
    }
    int read(const Entry &t, void *dst) {
        ShardFile &s = shards[(size_t)t.shard];
        if (s.fd < 0) {
            s.fd = open(s.path.c_str(), O_RDONLY);
            if (s.fd < 0) return fail(MUMMU_ERR_IO, s.path + ": cannot open: " + strerror(errno));
        }
        uint64_t done = 0;
        const uint64_t n = t.end - t.start;
        while (done < n) {
            const ssize_t got = pread(s.fd, (char *)dst + done, (size_t)std::min<uint64_t>(n - done, 1u << 30), (off_t)(s.data_offset + t.start + done));
            if (got <= 0) return fail(MUMMU_ERR_IO, s.path + ": short read of tensor '" + t.name + "'");
            done += (uint64_t)got;
        }
        return MUMMU_OK;
    }
};

namespace {

// One layer's tensors located and checked (nothing read): router, norm (or -1) and the three
// groups of E members in numeric expert order.
struct LayerPlan {
    int router = -1, norm = -1;
    std::vector<int> gate, up, down;
};

int plan_layer(const mummu_st *st, const mummu_moe_config &c, int layer, LayerPlan &plan) {
    const std::string base = "model.layers." + std::to_string(layer) + ".";
    const uint64_t H = (uint64_t)c.hidden_size, I = (uint64_t)c.expert_intermediate_size, E = (uint64_t)c.num_experts;
    auto find = [&](const std::string &name) {
        const auto it = st->by_name.find(name);
        return it == st->by_name.end() ? -1 : it->second;
    };
    auto want_shape = [&](int idx, std::vector<uint64_t> shape) {
        const Entry &t = st->tensors[(size_t)idx];
        if (t.shape != shape) {
            std::string got = "[", want = "[";
            for (size_t i = 0; i < t.shape.size(); i++) got += (i ? ", " : "") + std::to_string(t.shape[i]);
            for (size_t i = 0; i < shape.size(); i++) want += (i ? ", " : "") + std::to_string(shape[i]);
            return fail(MUMMU_ERR_SHAPE, t.name + ": shape " + got + "] does not match the config's " + want + "]");
        }
        if (ggml_type_of(t.dtype) < 0) return fail(MUMMU_ERR_TYPE, t.name + ": dtype " + t.dtype + " is not a float type this loader takes (F32, F16, BF16)");
        return (int)MUMMU_OK;
    };
    int rc;
    plan.router = find(base + "mlp.gate.weight");
    if (plan.router < 0) return fail(MUMMU_ERR_SAFETENSORS, "checkpoint has no " + base + "mlp.gate.weight");
    if ((rc = want_shape(plan.router, {E, H}))) return rc;
    plan.norm = find(base + "post_attention_layernorm.weight");
    if (plan.norm >= 0 && (rc = want_shape(plan.norm, {H}))) return rc;
    // the groups: every member present exactly once, all of one dtype and shape
    struct Group {
        const char *proj;
        std::vector<int> *members;
        std::vector<uint64_t> shape;
    } groups[3] = {{"gate", &plan.gate, {I, H}}, {"up", &plan.up, {I, H}}, {"down", &plan.down, {H, I}}};
    for (Group &g : groups) {
        const std::string target = base + "mlp.experts." + g.proj;
        g.members->assign((size_t)E, -1);
        size_t present = 0;
        for (uint64_t i = 0; i < E; i++) {
            const int idx = find(base + "mlp.experts." + std::to_string(i) + "." + g.proj + "_proj.weight");
            (*g.members)[(size_t)i] = idx;
            present += idx >= 0;
        }
        // a member index outside 0..count (safetensors.rs:626-633)
        const std::string stray = base + "mlp.experts." + std::to_string(E) + "." + g.proj + "_proj.weight";
        if (find(stray) >= 0) return fail(MUMMU_ERR_SAFETENSORS, target + ": member index " + std::to_string(E) + " outside 0.." + std::to_string(E));
        if (present != E)
            return fail(MUMMU_ERR_SAFETENSORS, target + ": " + std::to_string(present) + " of " + std::to_string(E) +
                                                   " members present - a short group would load clean and compute wrong");
        const Entry &first = st->tensors[(size_t)(*g.members)[0]];
        for (int idx : *g.members) {
            const Entry &t = st->tensors[(size_t)idx];
            if (t.dtype != first.dtype || t.shape != first.shape)
                return fail(MUMMU_ERR_SAFETENSORS, target + ": members disagree on layout (" + first.name + " is " + first.dtype + ", " + t.name + " is " + t.dtype + " or of another shape)");
            if (t.end - t.start > kMaxPartBytes) return fail(MUMMU_ERR_SAFETENSORS, t.name + ": a single member exceeds 4 GiB");
        }
        if ((rc = want_shape((*g.members)[0], g.shape))) return rc;
    }
    if (st->tensors[(size_t)plan.gate[0]].dtype != st->tensors[(size_t)plan.up[0]].dtype)
        return fail(MUMMU_ERR_TYPE, base + "mlp.experts: gate and up projections must share one dtype");
    return MUMMU_OK;
}

float to_f32(const uint8_t *p, int ggml_type, size_t i) {
    if (ggml_type == MUMMU_F32) {
        float v;
        memcpy(&v, p + 4 * i, 4);
        return v;
    }
    uint16_t h;
    memcpy(&h, p + 2 * i, 2);
    uint32_t bits;
    if (ggml_type == MUMMU_BF16) {
        bits = (uint32_t)h << 16;
    } else {  // IEEE half, exact
        const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31u, man = h & 1023u;
        if (exp == 0) {
            if (man == 0) bits = sign;
            else {
                int e = -1;
                uint32_t m = man;
                do { e++; m <<= 1; } while (!(m & 1024u));
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 1023u) << 13);
            }
        } else if (exp == 31) {
            bits = sign | 0x7F800000u | (man << 13);
        } else {
            bits = sign | ((exp + 112u) << 23) | (man << 13);
        }
    }
    float v;
    memcpy(&v, &bits, 4);
    return v;
}

}  // namespace

extern "C" {

const char *mummu_st_last_error(void) { return g_st_error.c_str(); }

int mummu_olmoe_config_from_json(const char *json, size_t len, mummu_moe_config *cfg) {
    if (!json || !cfg) return fail(MUMMU_ERR_ARG, "null argument");
    Json j;
    std::string err;
    if (!JsonParser(json, len).parse(j, err)) return fail(MUMMU_ERR_CONFIG, "olmoe config.json: " + err);
    return config_from_json(j, "olmoe config.json", cfg);
}

int mummu_st_open(const char *dir_c, mummu_st **out) {
    if (!dir_c || !out) return fail(MUMMU_ERR_ARG, "null path or output pointer");
    *out = nullptr;
    std::string dir = dir_c;
    while (dir.size() > 1 && dir.back() == '/') dir.pop_back();
    // safetensors.rs:377-430
    std::vector<std::string> paths;
    if (is_file(dir + "/model.safetensors")) {
        paths.push_back(dir + "/model.safetensors");
    } else {
        const std::string index_path = dir + "/model.safetensors.index.json";
        if (!is_file(index_path)) return fail(MUMMU_ERR_IO, dir + ": holds neither model.safetensors nor model.safetensors.index.json");
        std::string text, err;
        if (!read_file(index_path, text, err)) return fail(MUMMU_ERR_IO, err);
        Json idx;
        if (!JsonParser(text.data(), text.size()).parse(idx, err)) return fail(MUMMU_ERR_SAFETENSORS, index_path + ": bad index: " + err);
        const Json *map = idx.get("weight_map");
        if (!map || map->kind != Json::Obj) return fail(MUMMU_ERR_SAFETENSORS, index_path + ": bad index: no weight_map object");
        std::vector<std::string> names;
        for (const auto &kv : map->obj) {
            if (kv.second.kind != Json::Str) return fail(MUMMU_ERR_SAFETENSORS, index_path + ": bad index: weight_map['" + kv.first + "'] is not a file name");
            const std::string &n = kv.second.str;
            if (n.empty() || n.find('/') != std::string::npos || n.find('\\') != std::string::npos || n == "." || n == "..")
                return fail(MUMMU_ERR_SAFETENSORS, index_path + ": bad index: shard name '" + n + "' is not a plain file name");
            if (std::find(names.begin(), names.end(), n) == names.end()) names.push_back(n);
        }
        std::sort(names.begin(), names.end());
        if (names.empty() || names.size() > kMaxShards)
            return fail(MUMMU_ERR_SAFETENSORS, index_path + ": bad index: names " + std::to_string(names.size()) + " shards (1..=" + std::to_string(kMaxShards) + ")");
        for (const std::string &n : names) {
            const std::string p = dir + "/" + n;
            if (!is_file(p)) {
                const bool part = is_file(p + ".part");
                return fail(MUMMU_ERR_IO, dir + ": missing shard " + n + (part ? " - a .part sibling is present, so the download was interrupted" : ""));
            }
            paths.push_back(p);
        }
    }
    std::unique_ptr<mummu_st> st(new mummu_st());
    st->dir = dir;
    st->shards.resize(paths.size());
    for (size_t s = 0; s < paths.size(); s++) {
        const int rc = parse_shard(paths[s], (int)s, st->shards[s], st->tensors);
        if (rc) return rc;
    }
    for (size_t i = 0; i < st->tensors.size(); i++)
        if (!st->by_name.emplace(st->tensors[i].name, (int)i).second)
            return fail(MUMMU_ERR_SAFETENSORS, dir + ": tensor '" + st->tensors[i].name + "' appears in more than one shard");
    // config.json is read here and judged when asked for
    const std::string cfg_path = dir + "/config.json";
    std::string text, err;
    if (!is_file(cfg_path) || !read_file(cfg_path, text, err)) {
        st->cfg_status = MUMMU_ERR_IO;
        st->cfg_error = dir + ": no readable config.json";
    } else {
        Json j;
        if (!JsonParser(text.data(), text.size()).parse(j, err)) {
            st->cfg_status = MUMMU_ERR_CONFIG;
            st->cfg_error = cfg_path + ": " + err;
        } else {
            st->cfg_status = config_from_json(j, cfg_path, &st->cfg);
            st->cfg_error = g_st_error;
            st->have_cfg = st->cfg_status == MUMMU_OK;
        }
    }
    g_st_error.clear();
    *out = st.release();
    return MUMMU_OK;
}

void mummu_st_close(mummu_st *st) { delete st; }
int mummu_st_shard_count(const mummu_st *st) { return st ? (int)st->shards.size() : -1; }
int mummu_st_tensor_count(const mummu_st *st) { return st ? (int)st->tensors.size() : -1; }

int mummu_st_find_tensor(const mummu_st *st, const char *name) {
    if (!st || !name) return -1;
    const auto it = st->by_name.find(name);
    return it == st->by_name.end() ? -1 : it->second;
}

int mummu_st_tensor_info(const mummu_st *st, int index, mummu_st_tensor *out) {
    if (!st || !out) return fail(MUMMU_ERR_ARG, "null argument");
    if (index < 0 || index >= (int)st->tensors.size()) return fail(MUMMU_ERR_RANGE, "tensor index " + std::to_string(index) + " out of range");
    const Entry &t = st->tensors[(size_t)index];
    out->name = t.name.c_str();
    out->dtype = t.dtype.c_str();
    out->n_dims = (int32_t)std::min<size_t>(t.shape.size(), 8);
    for (int i = 0; i < 8; i++) out->dims[i] = i < (int)t.shape.size() ? (int64_t)t.shape[(size_t)i] : 1;
    out->shard = t.shard;
    out->file_offset = st->shards[(size_t)t.shard].data_offset + t.start;
    out->nbytes = t.end - t.start;
    out->path = st->shards[(size_t)t.shard].path.c_str();
    return MUMMU_OK;
}

int mummu_st_moe_config(const mummu_st *st, mummu_moe_config *cfg) {
    if (!st || !cfg) return fail(MUMMU_ERR_ARG, "null argument");
    if (!st->have_cfg) return fail(st->cfg_status, st->cfg_error);
    *cfg = st->cfg;
    return MUMMU_OK;
}

int mummu_st_check_moe_layer(const mummu_st *st, int layer) {
    if (!st) return fail(MUMMU_ERR_ARG, "null argument");
    if (!st->have_cfg) return fail(st->cfg_status, st->cfg_error);
    if (layer < 0 || layer >= st->cfg.num_layers)
        return fail(MUMMU_ERR_RANGE, "layer " + std::to_string(layer) + " is not inside the checkpoint's " + std::to_string(st->cfg.num_layers) + " layers");
    LayerPlan plan;
    return plan_layer(st, st->cfg, layer, plan);
}

int mummu_moe_load_safetensors(mummu_moe *h, mummu_st *st, int first_layer, int n_layers) {
    if (!h || !st) return fail(MUMMU_ERR_ARG, "null argument");
    if (!st->have_cfg) return fail(st->cfg_status, st->cfg_error);
    if (first_layer < 0 || n_layers < 1) return fail(MUMMU_ERR_RANGE, "first_layer must be >= 0 and n_layers >= 1");
    const mummu_moe_config &c = st->cfg;
    {
        // the handle reads its banks by its own geometry: a checkpoint of another geometry would be read past its buffers
        mummu_moe_config have;
        const int rc = mummu_moe_get_config(h, &have);
        if (rc) return fail(rc, "the handle's configuration could not be read");
        if (have.hidden_size != c.hidden_size || have.expert_intermediate_size != c.expert_intermediate_size || have.num_experts != c.num_experts)
            return fail(MUMMU_ERR_SHAPE, "the handle was created for hidden " + std::to_string(have.hidden_size) + ", intermediate " +
                                             std::to_string(have.expert_intermediate_size) + ", " + std::to_string(have.num_experts) +
                                             " experts; the checkpoint holds hidden " + std::to_string(c.hidden_size) + ", intermediate " +
                                             std::to_string(c.expert_intermediate_size) + ", " + std::to_string(c.num_experts) + " experts");
        if (n_layers > have.num_layers)
            return fail(MUMMU_ERR_RANGE, std::to_string(n_layers) + " layers do not fit the handle's " + std::to_string(have.num_layers));
    }
    std::vector<uint8_t> router, banks[3];
    std::vector<float> gamma;
    for (int l = 0; l < n_layers; l++) {
        const int layer = first_layer + l;
        if (layer >= c.num_layers)
            return fail(MUMMU_ERR_RANGE, "layer " + std::to_string(layer) + " is not inside the checkpoint's " + std::to_string(c.num_layers) + " layers");
        LayerPlan plan;
        int rc = plan_layer(st, c, layer, plan);
        if (rc) return rc;
        const Entry &r = st->tensors[(size_t)plan.router];
        router.resize((size_t)(r.end - r.start));
        if ((rc = st->read(r, router.data()))) return rc;
        // the fuse: members stacked along a new leading axis in numeric expert order
        const std::vector<int> *groups[3] = {&plan.gate, &plan.up, &plan.down};
        int types[3];
        for (int g = 0; g < 3; g++) {
            const Entry &first = st->tensors[(size_t)(*groups[g])[0]];
            const size_t each = (size_t)(first.end - first.start);
            types[g] = ggml_type_of(first.dtype);
            banks[g].resize(each * groups[g]->size());
            for (size_t e = 0; e < groups[g]->size(); e++)
                if ((rc = st->read(st->tensors[(size_t)(*groups[g])[e]], banks[g].data() + e * each))) return rc;
        }
        const float *gamma_ptr = nullptr;
        if (plan.norm >= 0) {
            const Entry &n = st->tensors[(size_t)plan.norm];
            std::vector<uint8_t> raw((size_t)(n.end - n.start));
            if ((rc = st->read(n, raw.data()))) return rc;
            gamma.resize((size_t)c.hidden_size);
            const int t = ggml_type_of(n.dtype);
            for (size_t i = 0; i < gamma.size(); i++) gamma[i] = to_f32(raw.data(), t, i);
            gamma_ptr = gamma.data();
        }
        rc = mummu_moe_load_layer(h, l, router.data(), ggml_type_of(r.dtype), banks[0].data(), types[0], banks[1].data(), types[1],
                                  banks[2].data(), types[2], gamma_ptr);
        if (rc) return fail(rc, "model.layers." + std::to_string(layer) + ": " + mummu_moe_last_error(h));
    }
    g_st_error.clear();
    return MUMMU_OK;
}

}  // extern "C"
