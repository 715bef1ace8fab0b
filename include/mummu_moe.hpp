// mummu_moe.hpp - C++ host side above the C ABI of mummu_moe.h.
//
// Mirrors the reference's module interface for the sparse MoE block (physics515/Mummu, paths
// under crates/mummu/src/): the same type and method names, argument meaning and error
// behaviour, so that a caller written against the Rust API reads the same here.
//
//   reference                                         here
//   SparseMoeConfig            nn/moe.rs:42-50        mummu::SparseMoeConfig
//   SparseMoe::forward         nn/moe.rs:116          mummu::SparseMoe::forward
//   SparseMoePerExpert::route  nn/moe.rs:247-290      mummu::SparseMoe::route -> mummu::Routing
//   SparseMoePerExpert::run_local nn/moe.rs:296-328   mummu::SparseMoe::run_local
//   Routing                    nn/moe.rs:333-337      mummu::Routing (per_expert rows + weights)
//   ExpertExec                 nn/moe.rs:348-419      mummu::ExpertExec, mummu::HipExpert
//   RoutedExperts::routed_moe / apply_routing / expert_ffn
//                              models/qwen4exp/experts.rs:1015-1150
//                                                      mummu::RoutedExperts
//   route                      experts.rs:541-582     mummu::route
//   gguf::dequantize           gguf.rs:1403-1463      mummu::dequantize
//   GgufFile::open_sharded, tensor, get, payload_location
//                              gguf.rs:577-714, 1062-1122
//                                                      mummu::GgufFile
//   OlmoeConfig::from_gguf (MoE fields) models/olmoe.rs:116-179   mummu::GgufFile::moe_config
//   RoutedExperts::open (bank locator) experts.rs:869-911         mummu::GgufFile::locate_moe_layer,
//                                                                  mummu::SparseMoe::from_gguf
//   OlmoeConfig::from_json_bytes  models/olmoe.rs:104-108          mummu::olmoe_config_from_json
//   checkpoint_shards, SafetensorsHeader::open, olmoe_hf_fuse, load_from_dir
//                              safetensors.rs:180-430; models/olmoe.rs:405-500
//                                                      mummu::Checkpoint, mummu::SparseMoe::from_checkpoint
//
// Error behaviour: the reference panics on contract violations of SparseMoe (assert!) and
// returns Err(String) from the qwen4exp functions.  Both surface here as mummu::MoeError (a
// std::runtime_error carrying the status code and the library's message); nothing is swallowed.
// Header-only; link with -lmummu_moe.
#pragma once

#include <cstdint>
#include <limits>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "mummu_moe.h"

namespace mummu {

class MoeError : public std::runtime_error {
  public:
    MoeError(int status, const std::string &msg) : std::runtime_error(msg), status_(status) {}
    int status() const { return status_; }

  private:
    int status_;
};

// SparseMoeConfig (nn/moe.rs:42-50) plus the OlmoeConfig fields the block reads
// (models/olmoe.rs:52-66).
struct SparseMoeConfig {
    int hidden_size = 0;
    int expert_intermediate_size = 0;
    int num_experts = 0;
    int num_experts_per_tok = 0;
    bool norm_topk_prob = false;
    int router_flavour = MUMMU_ROUTER_SPARSE_MOE;
    int num_layers = 1;
    int max_tokens = 512;
    float rms_norm_eps = 1e-5f;
};

// One GGUF tensor payload: host bytes in GGUF order plus its ggml type id.
struct TensorBytes {
    const void *data = nullptr;
    int ggml_type = MUMMU_F32;
};

// Routing (nn/moe.rs:333-337): per expert, the token rows it serves (ascending, token-major
// slot-minor fill) and the matching combine weights; plus the slot-ordered form.
struct Routing {
    int64_t tokens = 0;
    int top_k = 0;
    std::vector<int32_t> ids;      // [tokens, top_k], descending probability
    std::vector<float> weights;    // [tokens, top_k]
    std::vector<std::pair<std::vector<int32_t>, std::vector<float>>> per_expert;

    static Routing from_slots(std::vector<int32_t> ids, std::vector<float> weights, int64_t tokens, int top_k,
                              int num_experts) {
        Routing r;
        r.tokens = tokens;
        r.top_k = top_k;
        r.per_expert.resize((size_t)num_experts);
        for (int64_t t = 0; t < tokens; t++)
            for (int s = 0; s < top_k; s++) {
                const int32_t e = ids[(size_t)(t * top_k + s)];
                if (e < 0 || e >= num_experts) throw MoeError(MUMMU_ERR_RANGE, "routing names expert " + std::to_string(e));
                r.per_expert[(size_t)e].first.push_back((int32_t)t);
                r.per_expert[(size_t)e].second.push_back(weights[(size_t)(t * top_k + s)]);
            }
        r.ids = std::move(ids);
        r.weights = std::move(weights);
        return r;
    }
};

// GgufError (gguf.rs:65-118): every refusal of the container reader.
class GgufError : public MoeError {
  public:
    using MoeError::MoeError;
};

// GgufTensorInfo (gguf.rs:403-430) with its payload location (gguf.rs:1096).
struct GgufTensorInfo {
    std::string name;
    std::vector<uint64_t> dims;  // GGUF order, fastest-varying first
    int ggml_type = 0;
    int shard = 0;
    std::string path;
    uint64_t file_offset = 0;
    uint64_t byte_len = 0;
};

// A parsed and validated GGUF file or split set (gguf.rs:538-714).
class GgufFile {
  public:
    // GgufFile::open_sharded (gguf.rs:628): a single file, or any member of a split set.
    static GgufFile open(const std::string &path) {
        mummu_gguf *g = nullptr;
        const int rc = mummu_gguf_open(path.c_str(), &g);
        if (rc != MUMMU_OK) throw GgufError(rc, mummu_gguf_last_error());
        return GgufFile(g);
    }
    mummu_gguf *handle() const { return g_.get(); }
    int version() const { return mummu_gguf_version(g_.get()); }
    uint64_t alignment() const { return (uint64_t)mummu_gguf_alignment(g_.get()); }
    size_t shard_count() const { return (size_t)mummu_gguf_shard_count(g_.get()); }
    size_t tensor_count() const { return (size_t)mummu_gguf_tensor_count(g_.get()); }
    std::optional<std::string> architecture() const { return get_str("general.architecture"); }

    std::optional<uint64_t> get_u64(const std::string &key) const {
        uint64_t v = 0;
        if (mummu_gguf_get_u64(g_.get(), key.c_str(), &v) != MUMMU_OK) return std::nullopt;
        return v;
    }
    std::optional<double> get_f64(const std::string &key) const {
        double v = 0;
        if (mummu_gguf_get_f64(g_.get(), key.c_str(), &v) != MUMMU_OK) return std::nullopt;
        return v;
    }
    std::optional<std::string> get_str(const std::string &key) const {
        const char *s = mummu_gguf_get_str(g_.get(), key.c_str());
        if (!s) return std::nullopt;
        return std::string(s);
    }

    std::optional<size_t> tensor_index(const std::string &name) const {
        const int i = mummu_gguf_find_tensor(g_.get(), name.c_str());
        if (i < 0) return std::nullopt;
        return (size_t)i;
    }
    GgufTensorInfo tensor_at(size_t index) const {
        mummu_gguf_tensor t{};
        check(mummu_gguf_tensor_info(g_.get(), (int)index, &t));
        GgufTensorInfo out;
        out.name = t.name;
        out.dims.assign(t.dims, t.dims + t.n_dims);
        out.ggml_type = t.ggml_type;
        out.shard = t.shard;
        out.path = t.path;
        out.file_offset = t.file_offset;
        out.byte_len = t.nbytes;
        return out;
    }
    std::optional<GgufTensorInfo> tensor(const std::string &name) const {
        const auto i = tensor_index(name);
        if (!i) return std::nullopt;
        return tensor_at(*i);
    }
    // The payload bytes, mapped read-only; valid while this object lives.
    std::pair<const uint8_t *, uint64_t> tensor_bytes(const std::string &name) const {
        const auto i = tensor_index(name);
        if (!i) throw GgufError(MUMMU_ERR_GGUF, "GGUF has no " + name);
        const void *p = nullptr;
        uint64_t n = 0;
        check(mummu_gguf_tensor_data(g_.get(), (int)*i, &p, &n));
        return {(const uint8_t *)p, n};
    }

    // The MoE fields of OlmoeConfig::from_gguf (models/olmoe.rs:116-179).
    SparseMoeConfig moe_config() const {
        mummu_moe_config k{};
        check(mummu_gguf_moe_config(g_.get(), &k));
        SparseMoeConfig c;
        c.hidden_size = k.hidden_size;
        c.expert_intermediate_size = k.expert_intermediate_size;
        c.num_experts = k.num_experts;
        c.num_experts_per_tok = k.num_experts_per_tok;
        c.norm_topk_prob = k.norm_topk_prob != 0;
        c.router_flavour = k.router_flavour;
        c.num_layers = k.num_layers;
        c.max_tokens = k.max_tokens;
        c.rms_norm_eps = k.rms_norm_eps;
        return c;
    }
    // The bank locator for one layer (experts.rs:869-911): tensor indices, norm -1 when absent.
    mummu_gguf_moe_layer locate_moe_layer(int layer) const {
        mummu_gguf_moe_layer at{};
        check(mummu_gguf_locate_moe_layer(g_.get(), layer, &at));
        return at;
    }

  private:
    explicit GgufFile(mummu_gguf *g) : g_(g, mummu_gguf_close) {}
    static void check(int rc) {
        if (rc != MUMMU_OK) throw GgufError(rc, mummu_gguf_last_error());
    }
    std::shared_ptr<mummu_gguf> g_;
};

// SafetensorsError (safetensors.rs:62-118) and the config errors of OlmoeConfig::from_json_bytes.
class SafetensorsError : public MoeError {
  public:
    using MoeError::MoeError;
};

inline SparseMoeConfig moe_config_of(const mummu_moe_config &k) {
    SparseMoeConfig c;
    c.hidden_size = k.hidden_size;
    c.expert_intermediate_size = k.expert_intermediate_size;
    c.num_experts = k.num_experts;
    c.num_experts_per_tok = k.num_experts_per_tok;
    c.norm_topk_prob = k.norm_topk_prob != 0;
    c.router_flavour = k.router_flavour;
    c.num_layers = k.num_layers;
    c.max_tokens = k.max_tokens;
    c.rms_norm_eps = k.rms_norm_eps;
    return c;
}

// OlmoeConfig::from_json_bytes (models/olmoe.rs:104-108): the MoE block's fields, validated.
inline SparseMoeConfig olmoe_config_from_json(const std::string &json) {
    mummu_moe_config k{};
    const int rc = mummu_olmoe_config_from_json(json.data(), json.size(), &k);
    if (rc != MUMMU_OK) throw SafetensorsError(rc, mummu_st_last_error());
    return moe_config_of(k);
}

// An HF safetensors checkpoint directory (safetensors.rs:180-430): shards discovered and every
// header entry validated on open.
class Checkpoint {
  public:
    static Checkpoint open(const std::string &dir) {
        mummu_st *st = nullptr;
        const int rc = mummu_st_open(dir.c_str(), &st);
        if (rc != MUMMU_OK) throw SafetensorsError(rc, mummu_st_last_error());
        return Checkpoint(st);
    }
    mummu_st *handle() const { return st_.get(); }
    size_t shard_count() const { return (size_t)mummu_st_shard_count(st_.get()); }
    size_t tensor_count() const { return (size_t)mummu_st_tensor_count(st_.get()); }
    std::optional<mummu_st_tensor> tensor(const std::string &name) const {
        const int i = mummu_st_find_tensor(st_.get(), name.c_str());
        if (i < 0) return std::nullopt;
        mummu_st_tensor t{};
        check(mummu_st_tensor_info(st_.get(), i, &t));
        return t;
    }
    SparseMoeConfig moe_config() const {
        mummu_moe_config k{};
        check(mummu_st_moe_config(st_.get(), &k));
        return moe_config_of(k);
    }
    // The fuse's planning pass for one layer (olmoe_hf_fuse + the group rules), nothing read.
    void check_moe_layer(int layer) const { check(mummu_st_check_moe_layer(st_.get(), layer)); }

  private:
    explicit Checkpoint(mummu_st *st) : st_(st, mummu_st_close) {}
    static void check(int rc) {
        if (rc != MUMMU_OK) throw SafetensorsError(rc, mummu_st_last_error());
    }
    std::shared_ptr<mummu_st> st_;
};

// The block, resident on the MI355X.  One object holds every MoE layer of a model.
class SparseMoe {
  public:
    explicit SparseMoe(const SparseMoeConfig &c) : cfg_(c) {
        mummu_moe_config k{};
        k.hidden_size = c.hidden_size;
        k.expert_intermediate_size = c.expert_intermediate_size;
        k.num_experts = c.num_experts;
        k.num_experts_per_tok = c.num_experts_per_tok;
        k.norm_topk_prob = c.norm_topk_prob ? 1 : 0;
        k.router_flavour = c.router_flavour;
        k.num_layers = c.num_layers;
        k.max_tokens = c.max_tokens;
        k.rms_norm_eps = c.rms_norm_eps;
        mummu_moe *h = nullptr;
        const int rc = mummu_moe_create(&k, &h);
        if (rc != MUMMU_OK) throw MoeError(rc, mummu_moe_last_error(nullptr));
        h_.reset(h, mummu_moe_destroy);
    }

    const SparseMoeConfig &config() const { return cfg_; }
    mummu_moe *handle() const { return h_.get(); }

    // The checked load of one block (models/olmoe.rs:338-345).
    void load_layer(int layer, TensorBytes router, TensorBytes gate, TensorBytes up, TensorBytes down,
                    const float *rms_gamma = nullptr) {
        check(mummu_moe_load_layer(h_.get(), layer, router.data, router.ggml_type, gate.data, gate.ggml_type, up.data,
                                   up.ggml_type, down.data, down.ggml_type, rms_gamma));
    }

    // The MoE blocks of file layers [first_layer, first_layer + n_layers) as layers 0.. of a new
    // object, payload bytes unchanged (RoutedExperts::open, experts.rs:869-911).  n_layers < 0
    // takes every layer from first_layer on.
    static SparseMoe from_gguf(const GgufFile &f, int first_layer = 0, int n_layers = -1, int max_tokens = 512,
                               int router_flavour = MUMMU_ROUTER_SPARSE_MOE) {
        SparseMoeConfig c = f.moe_config();
        if (n_layers < 0) n_layers = c.num_layers - first_layer;
        c.num_layers = n_layers > 0 ? n_layers : 1;
        c.max_tokens = max_tokens;
        c.router_flavour = router_flavour;
        SparseMoe m(c);
        const int rc = mummu_moe_load_gguf(m.handle(), f.handle(), first_layer, n_layers);
        if (rc != MUMMU_OK) throw GgufError(rc, mummu_gguf_last_error());
        return m;
    }

    // The same from an HF checkpoint directory: per-expert projections fused into [E, out, in]
    // banks of the stored dtype (load_from_dir, models/olmoe.rs:432-500).
    static SparseMoe from_checkpoint(const Checkpoint &ck, int first_layer = 0, int n_layers = -1, int max_tokens = 512) {
        SparseMoeConfig c = ck.moe_config();
        if (n_layers < 0) n_layers = c.num_layers - first_layer;
        c.num_layers = n_layers > 0 ? n_layers : 1;
        c.max_tokens = max_tokens;
        SparseMoe m(c);
        const int rc = mummu_moe_load_safetensors(m.handle(), ck.handle(), first_layer, n_layers);
        if (rc != MUMMU_OK) throw SafetensorsError(rc, mummu_st_last_error());
        return m;
    }

    // The shared expert of a Qwen-style block and its sigmoid gate vector (may be null)
    // (models/qwen4exp/model.rs:786-804): forward then returns routed + shared(x) * sigmoid(<gate_vec, x>).
    void load_shared_expert(int layer, int inter, TensorBytes gate, TensorBytes up, TensorBytes down,
                            TensorBytes gate_vec = TensorBytes()) {
        check(mummu_moe_load_shared_expert(h_.get(), layer, inter, gate.data, gate.ggml_type, up.data, up.ggml_type, down.data,
                                           down.ggml_type, gate_vec.data, gate_vec.ggml_type));
    }

    uint64_t resident_bytes() const { return mummu_moe_resident_bytes(h_.get()); }
    /// The configuration as the handle holds it (mummu_moe_get_config).
    mummu_moe_config handle_config() const {
        mummu_moe_config c{};
        mummu_moe_get_config(h_.get(), &c);
        return c;
    }
    /// Smallest token count that takes dispatch + grouped GEMM on this layer (INT32_MAX: never).
    int batched_from(int layer = 0) const { return mummu_moe_batched_from(h_.get(), layer); }

    // SparseMoe::forward (nn/moe.rs:116): x [tokens, hidden] -> [tokens, hidden].
    std::vector<float> forward(const std::vector<float> &x, int top_k, bool norm_topk_prob, int layer = 0) {
        const int64_t n = rows_of(x);
        std::vector<float> out(x.size());
        check(mummu_moe_forward(h_.get(), layer, x.data(), n, top_k, norm_topk_prob ? 1 : 0, out.data()));
        return out;
    }

    // SparseMoePerExpert::route (nn/moe.rs:247-290).
    Routing route(const std::vector<float> &x, int top_k, bool norm_topk_prob, int layer = 0) {
        const int64_t n = rows_of(x);
        std::vector<int32_t> ids((size_t)(n * top_k));
        std::vector<float> w((size_t)(n * top_k));
        check(mummu_moe_route(h_.get(), layer, x.data(), n, top_k, norm_topk_prob ? 1 : 0, ids.data(), w.data(), nullptr));
        return Routing::from_slots(std::move(ids), std::move(w), n, top_k, cfg_.num_experts);
    }

    // SparseMoePerExpert::run_local (nn/moe.rs:296-328) / ExpertPool::run_layer (:1545-1607).
    std::vector<float> run_local(const std::vector<float> &x, const Routing &routing, int layer = 0) {
        const int64_t n = rows_of(x);
        if (n != routing.tokens) throw MoeError(MUMMU_ERR_SHAPE, "routing was made for a different token count");
        std::vector<float> out(x.size());
        check(mummu_moe_apply_routing(h_.get(), layer, routing.ids.data(), routing.weights.data(), x.data(), n, routing.top_k,
                                      out.data()));
        return out;
    }

    // ExpertPool::take_hits (nn/moe.rs:857-874).
    std::vector<uint64_t> take_hits(int layer = 0) {
        std::vector<uint64_t> hits((size_t)cfg_.num_experts);
        check(mummu_moe_take_hits(h_.get(), layer, hits.data()));
        return hits;
    }

    // x <- x + MoE_l(RmsNorm_l(x)) over every layer (models/olmoe.rs:566-572).
    std::vector<float> stack_forward(const std::vector<float> &x, int top_k, bool norm_topk_prob) {
        const int64_t n = rows_of(x);
        std::vector<float> out(x.size());
        check(mummu_moe_stack_forward(h_.get(), x.data(), n, top_k, norm_topk_prob ? 1 : 0, out.data(), nullptr));
        return out;
    }

    // gguf::dequantize of one resident expert matrix (which: 0 gate, 1 up, 2 down).
    std::vector<float> dequantize_expert(int layer, int which, int expert) {
        const size_t n = (size_t)cfg_.hidden_size * (size_t)cfg_.expert_intermediate_size;
        std::vector<float> out(n);
        check(mummu_moe_dequantize_expert(h_.get(), layer, which, expert, out.data()));
        return out;
    }

    void check(int rc) const {
        if (rc != MUMMU_OK) throw MoeError(rc, mummu_moe_last_error(h_.get()));
    }

  private:
    int64_t rows_of(const std::vector<float> &x) const {
        if (cfg_.hidden_size <= 0 || x.size() % (size_t)cfg_.hidden_size != 0)
            throw MoeError(MUMMU_ERR_SHAPE, "input length is not a whole number of hidden-size rows");
        return (int64_t)(x.size() / (size_t)cfg_.hidden_size);
    }

    SparseMoeConfig cfg_;
    std::shared_ptr<mummu_moe> h_;
};

// SparseMoePerExpert (nn/moe.rs:202-329) has the same forward / route / run_local surface; on
// this device both are the routed kernels.
using SparseMoePerExpert = SparseMoe;

// ExpertExec (nn/moe.rs:348-419), the host-slice seam: SwiGLU of one expert on rows x hidden f32.
// Tier (tier.rs:66-71): the device an expert is placed on and the stored level it is loaded at (here: the GGML
// type of its gate bank).
struct Tier {
    int device = 0;
    int precision = MUMMU_F32;
};

class ExpertExec {
  public:
    virtual ~ExpertExec() = default;
    virtual Tier tier() const = 0;
    virtual std::vector<float> run(const float *x, size_t rows, size_t hidden) const = 0;
    virtual uint64_t resident_bytes() const = 0;
    // An executor pinned to its device is always resident there: staging and evicting it are no-ops, as the
    // trait's defaults are (nn/moe.rs:383-397); there is no second multiply path to fall back to either.
    virtual void stage(int /*device*/) const {}
    virtual void evict() const {}
    virtual bool is_staged() const { return true; }
    virtual void disable_native() const {}
    // Per-row energy of the gate activations; the default never skips (nn/moe.rs:411-418).
    virtual std::vector<float> gate_energy(const float * /*x*/, size_t rows, size_t /*hidden*/) const {
        return std::vector<float>(rows, std::numeric_limits<float>::infinity());
    }
};

// One expert of one layer of a SparseMoe, as an ExpertExec.
class HipExpert final : public ExpertExec {
  public:
    HipExpert(SparseMoe moe, int layer, int expert, int gate_type = MUMMU_F32)
        : moe_(std::move(moe)), layer_(layer), expert_(expert), gate_type_(gate_type) {}
    std::vector<float> run(const float *x, size_t rows, size_t hidden) const override {
        std::vector<float> out(rows * hidden);
        moe_.check(mummu_expert_run(moe_.handle(), layer_, expert_, x, (int64_t)rows, (int)hidden, out.data()));
        return out;
    }
    uint64_t resident_bytes() const override {
        const int e = moe_.config().num_experts * moe_.config().num_layers;
        return e > 0 ? moe_.resident_bytes() / (uint64_t)e : 0;
    }
    Tier tier() const override { return Tier{0, gate_type_}; }
    // run_tensor_resident (nn/moe.rs:360-371): rows already on this device, the result left there; only enqueues
    // on the handle's stream.
    void run_resident(const float *x_dev, size_t rows, size_t hidden, float *out_dev) const {
        moe_.check(mummu_expert_run_device(moe_.handle(), layer_, expert_, x_dev, (int64_t)rows, (int)hidden, out_dev,
                                           mummu_moe_stream(moe_.handle())));
    }
    std::vector<float> gate_energy(const float *x, size_t rows, size_t hidden) const override {
        std::vector<float> out(rows);
        moe_.check(mummu_expert_gate_energy(moe_.handle(), layer_, expert_, x, (int64_t)rows, (int)hidden, out.data()));
        return out;
    }

  private:
    SparseMoe moe_;
    int layer_, expert_, gate_type_;
};

// A weight in burn's packed block-32 layout behind Q4GemvOps::q4s_gemv (nn/packed_gemv.rs:248-260): words
// [K, N*bits/32] u32, scales [K, N/32] f32 (pack.rs:940-985), uploaded once.
class PackedWeight {
  public:
    PackedWeight(const std::vector<uint32_t> &words, const std::vector<float> &scales, int k, int n, int value_bits = 4)
        : k_(k), n_(n) {
        if (words.size() != (size_t)k * (size_t)n * (size_t)value_bits / 32 || scales.size() != (size_t)k * (size_t)(n / 32))
            throw MoeError(MUMMU_ERR_SHAPE, "packed weight: words / scales do not make [K, N] at this width");
        mummu_packed_weight *h = nullptr;
        const int rc = mummu_packed_weight_create(words.data(), scales.data(), k, n, value_bits, &h);
        if (rc != MUMMU_OK) throw MoeError(rc, mummu_packed_last_error());
        h_.reset(h, mummu_packed_weight_destroy);
    }
    // try_q4s_gemv (nn/packed_gemv.rs:98-152): x [m, K] -> [m, N], m <= 64.
    std::vector<float> gemv(const std::vector<float> &x) const {
        if (k_ <= 0 || x.size() % (size_t)k_ != 0) throw MoeError(MUMMU_ERR_SHAPE, "input length is not a whole number of K-wide rows");
        const size_t m = x.size() / (size_t)k_;
        std::vector<float> y(m * (size_t)n_);
        const int rc = mummu_q4s_gemv(h_.get(), x.data(), (int64_t)m, k_, y.data());
        if (rc != MUMMU_OK) throw MoeError(rc, mummu_packed_last_error());
        return y;
    }
    uint64_t resident_bytes() const { return mummu_packed_weight_bytes(h_.get()); }
    mummu_packed_weight *handle() const { return h_.get(); }

  private:
    int k_, n_;
    std::shared_ptr<mummu_packed_weight> h_;
};

// RoutedExperts (models/qwen4exp/experts.rs:1066-1150): caller-supplied router logits, qwen4exp
// routing rules (f64 normaliser, 2^-14 floor, non-finite logits refused).
class RoutedExperts {
  public:
    explicit RoutedExperts(SparseMoe moe) : moe_(std::move(moe)) {}

    std::vector<float> routed_moe(int layer, const std::vector<float> &router_logits, const std::vector<float> &xs, size_t n,
                                  int top_k) {
        std::vector<float> out(xs.size());
        moe_.check(mummu_moe_routed(moe_.handle(), layer, router_logits.data(), xs.data(), (int64_t)n, top_k, out.data()));
        return out;
    }

    std::vector<float> apply_routing(int layer, const std::vector<int32_t> &ids, const std::vector<float> &weights,
                                     const std::vector<float> &xs, size_t n, int top_k) {
        std::vector<float> out(xs.size());
        moe_.check(mummu_moe_apply_routing(moe_.handle(), layer, ids.data(), weights.data(), xs.data(), (int64_t)n, top_k,
                                           out.data()));
        return out;
    }

    std::vector<float> expert_ffn(int layer, int expert, const std::vector<float> &xs, size_t n) {
        std::vector<float> out(xs.size());
        moe_.check(mummu_expert_run(moe_.handle(), layer, expert, xs.data(), (int64_t)n, moe_.config().hidden_size, out.data()));
        return out;
    }

  private:
    SparseMoe moe_;
};

// `route` (experts.rs:541-582) on caller-supplied logits: (ids, weights), each [n, top_k].  The
// SparseMoe only lends its device workspace; no weights are involved and n_experts is free.
inline std::pair<std::vector<int32_t>, std::vector<float>> route(const SparseMoe &moe, const std::vector<float> &logits,
                                                                  size_t n, int n_experts, int top_k,
                                                                  int flavour = MUMMU_ROUTER_QWEN4EXP,
                                                                  bool norm_topk_prob = true) {
    std::vector<int32_t> ids(n * (size_t)top_k);
    std::vector<float> w(n * (size_t)top_k);
    moe.check(mummu_route_logits(moe.handle(), logits.data(), (int64_t)n, n_experts, top_k, flavour, norm_topk_prob ? 1 : 0,
                                 ids.data(), w.data()));
    return {std::move(ids), std::move(w)};
}

// gguf::dequantize (gguf.rs:1403-1463): payload bytes -> f32, bit-exact.
inline std::vector<float> dequantize(int ggml_type, const void *bytes, size_t nbytes, size_t n_elements) {
    std::vector<float> out(n_elements);
    const int rc = mummu_dequantize(ggml_type, bytes, nbytes, out.data());
    if (rc != MUMMU_OK) throw MoeError(rc, mummu_moe_last_error(nullptr));
    return out;
}

}  // namespace mummu
