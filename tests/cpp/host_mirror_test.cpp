// Exercises the C++ host mirror (include/mummu_moe.hpp) the way the reference's own unit tests
// exercise the Rust API, on the reference's closed-form toy block (nn/moe.rs:1617-1651):
//   forward_matches_the_hand_rolled_sparse_reference   nn/moe.rs:2177-2202
//   routed == fused forward, hits == tokens * top_k    nn/moe.rs:1655-1700, 1976-1979
//   zero input -> zero output                          nn/moe.rs:2340-2352
//   contract violations are loud                       nn/moe.rs:119-130
//   route known answers                                models/qwen4exp/experts.rs:1365-1388
//   GGUF reader: round trip, refusals, bank locator    gguf.rs:2280-2378, experts.rs:869-911
// `--no-gpu` runs only the checks that need no device (config validation, GGUF parsing).
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "mummu_moe.hpp"

static int failures = 0;
#define EXPECT(cond, what)                                         \
    do {                                                           \
        if (!(cond)) {                                             \
            std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, what); \
            failures++;                                            \
        }                                                          \
    } while (0)

static const int H = 4, I = 3, E = 4, K = 2;

// f32_from_usize(i).mul_add(0.37, seed).sin() * 0.5  (nn/moe.rs:1627-1629)
static std::vector<float> sin_fill(float seed, int n) {
    std::vector<float> v((size_t)n);
    for (int i = 0; i < n; i++) {
        const float arg = (float)((double)i * (double)0.37f + (double)seed);
        v[(size_t)i] = (float)std::sin((double)arg) * 0.5f;
    }
    return v;
}

// router stored [H,E] in the reference (nn/moe.rs:1642-1645); the ABI takes row-major [E,H].
static std::vector<float> router_eh() {
    std::vector<float> he((size_t)(H * E)), eh((size_t)(E * H));
    for (int i = 0; i < H * E; i++) he[(size_t)i] = (float)std::cos((double)(float)((double)i * (double)0.61f + 1.0)) * 0.5f;
    for (int h = 0; h < H; h++)
        for (int e = 0; e < E; e++) eh[(size_t)(e * H + h)] = he[(size_t)(h * E + e)];
    return eh;
}

// ((i + seed) * 0.9).sin()  (nn/moe.rs:2088-2093)
static std::vector<float> input(int t, float seed) {
    std::vector<float> x((size_t)(t * H));
    for (int i = 0; i < t * H; i++) x[(size_t)i] = (float)std::sin((double)(((float)i + seed) * 0.9f));
    return x;
}

// The hand-rolled scalar block of nn/moe.rs:2101-2175.
static std::vector<float> reference(const std::vector<float> &r, const std::vector<float> &g, const std::vector<float> &u,
                                    const std::vector<float> &d, const std::vector<float> &xs, int t, int top_k, bool norm) {
    std::vector<float> out((size_t)(t * H), 0.0f);
    for (int tok = 0; tok < t; tok++) {
        const float *x = &xs[(size_t)(tok * H)];
        float logits[E], probs[E];
        for (int e = 0; e < E; e++) {
            float s = 0.0f;
            for (int i = 0; i < H; i++) s += x[i] * r[(size_t)(e * H + i)];
            logits[e] = s;
        }
        float mx = logits[0];
        for (int e = 1; e < E; e++) mx = logits[e] > mx ? logits[e] : mx;
        float total = 0.0f;
        for (int e = 0; e < E; e++) {
            probs[e] = std::exp(logits[e] - mx);
            total += probs[e];
        }
        for (int e = 0; e < E; e++) probs[e] /= total;
        int order[E];
        for (int e = 0; e < E; e++) order[e] = e;
        for (int a = 1; a < E; a++)  // stable insertion sort, descending
            for (int b = a; b > 0 && probs[order[b]] > probs[order[b - 1]]; b--) std::swap(order[b], order[b - 1]);
        float denom = 1.0f;
        if (norm) {
            denom = 0.0f;
            for (int s = 0; s < top_k; s++) denom += probs[order[s]];
        }
        for (int s = 0; s < top_k; s++) {
            const int e = order[s];
            const float weight = probs[e] / denom;
            float act[I];
            for (int j = 0; j < I; j++) {
                float gg = 0.0f, uu = 0.0f;
                for (int i = 0; i < H; i++) {
                    gg += x[i] * g[(size_t)((e * I + j) * H + i)];
                    uu += x[i] * u[(size_t)((e * I + j) * H + i)];
                }
                act[j] = gg / (1.0f + std::exp(-gg)) * uu;
            }
            for (int i = 0; i < H; i++) {
                float dd = 0.0f;
                for (int j = 0; j < I; j++) dd += act[j] * d[(size_t)((e * H + i) * I + j)];
                out[(size_t)(tok * H + i)] += weight * dd;
            }
        }
    }
    return out;
}

template <typename F>
static bool throws(F &&f, int status, const char *needle) {
    try {
        f();
    } catch (const mummu::MoeError &e) {
        return e.status() == status && std::strstr(e.what(), needle) != nullptr;
    }
    return false;
}


// ---- a minimal GGUF v3 writer for the toy block (little-endian host) ---------------------------
struct GgufBytes {
    std::string head, payload;
    uint64_t n_kv = 0, n_tensors = 0;
    template <typename T>
    static void put(std::string &s, T v) {
        s.append((const char *)&v, sizeof(T));
    }
    static void put_str(std::string &s, const std::string &v) {
        put<uint64_t>(s, v.size());
        s += v;
    }
    std::string kvs, table;
    void kv_str(const std::string &k, const std::string &v) {
        put_str(kvs, k);
        put<uint32_t>(kvs, 8);
        put_str(kvs, v);
        n_kv++;
    }
    void kv_u32(const std::string &k, uint32_t v) {
        put_str(kvs, k);
        put<uint32_t>(kvs, 4);
        put<uint32_t>(kvs, v);
        n_kv++;
    }
    void kv_f32(const std::string &k, float v) {
        put_str(kvs, k);
        put<uint32_t>(kvs, 6);
        put<float>(kvs, v);
        n_kv++;
    }
    void tensor(const std::string &name, std::vector<uint64_t> dims, uint32_t type, const void *data, size_t nbytes) {
        payload.append((32 - payload.size() % 32) % 32, '\0');
        put_str(table, name);
        put<uint32_t>(table, (uint32_t)dims.size());
        for (uint64_t d : dims) put<uint64_t>(table, d);
        put<uint32_t>(table, type);
        put<uint64_t>(table, payload.size());
        payload.append((const char *)data, nbytes);
        n_tensors++;
    }
    std::string write(const std::string &name) const {
        std::string out = "GGUF";
        put<uint32_t>(out, 3);
        put<uint64_t>(out, n_tensors);
        put<uint64_t>(out, n_kv);
        out += kvs + table;
        out.append((32 - out.size() % 32) % 32, '\0');
        out += payload;
        const std::string path = "/tmp/mummu-host-mirror-" + std::to_string((long)getpid()) + "-" + name;
        FILE *f = std::fopen(path.c_str(), "wb");
        if (!f || std::fwrite(out.data(), 1, out.size(), f) != out.size()) {
            std::printf("FAIL cannot write %s\n", path.c_str());
            failures++;
        }
        if (f) std::fclose(f);
        return path;
    }
};

// The toy block as an OLMoE-named model file: router [H,E] in GGUF dims = row-major [E,H] bytes.
static GgufBytes toy_gguf(const std::vector<float> &r, const std::vector<float> &g, const std::vector<float> &u,
                          const std::vector<float> &d) {
    GgufBytes w;
    w.kv_str("general.architecture", "olmoe");
    w.kv_u32("olmoe.block_count", 1);
    w.kv_u32("olmoe.embedding_length", H);
    w.kv_u32("olmoe.feed_forward_length", I);
    w.kv_u32("olmoe.expert_count", E);
    w.kv_u32("olmoe.expert_used_count", K);
    w.kv_f32("olmoe.attention.layer_norm_rms_epsilon", 1e-5f);
    w.tensor("blk.0.ffn_gate_inp.weight", {H, E}, 0, r.data(), r.size() * 4);
    w.tensor("blk.0.ffn_gate_exps.weight", {H, I, E}, 0, g.data(), g.size() * 4);
    w.tensor("blk.0.ffn_up_exps.weight", {H, I, E}, 0, u.data(), u.size() * 4);
    w.tensor("blk.0.ffn_down_exps.weight", {I, H, E}, 0, d.data(), d.size() * 4);
    return w;
}

static void gguf_host_checks(const std::vector<float> &r, const std::vector<float> &g, const std::vector<float> &u,
                             const std::vector<float> &d) {
    const std::string path = toy_gguf(r, g, u, d).write("toy.gguf");
    {
        mummu::GgufFile f = mummu::GgufFile::open(path);
        EXPECT(f.version() == 3 && f.alignment() == 32 && f.shard_count() == 1 && f.tensor_count() == 4, "header fields");
        EXPECT(f.architecture() == std::optional<std::string>("olmoe"), "architecture");
        EXPECT(f.get_u64("olmoe.expert_count") == std::optional<uint64_t>(E), "typed metadata read");
        EXPECT(!f.get_u64("general.architecture") && !f.get_str("olmoe.expert_count") && !f.tensor("absent"), "absent or wrongly typed reads give nothing");
        const mummu::SparseMoeConfig c = f.moe_config();
        EXPECT(c.hidden_size == H && c.expert_intermediate_size == I && c.num_experts == E && c.num_experts_per_tok == K &&
                   c.num_layers == 1 && !c.norm_topk_prob,
               "MoE configuration from the header");
        const auto gate = f.tensor("blk.0.ffn_gate_exps.weight");
        EXPECT(gate && gate->dims == (std::vector<uint64_t>{H, I, E}) && gate->byte_len == (uint64_t)E * I * H * 4 && gate->file_offset % 32 == 0, "tensor info");
        const auto bytes = f.tensor_bytes("blk.0.ffn_down_exps.weight");
        EXPECT(bytes.second == d.size() * 4 && std::memcmp(bytes.first, d.data(), d.size() * 4) == 0, "payload bytes unchanged");
        const mummu_gguf_moe_layer at = f.locate_moe_layer(0);
        EXPECT(at.router >= 0 && at.gate >= 0 && at.up >= 0 && at.down >= 0 && at.norm == -1, "locator finds the four tensors, no norm");
        EXPECT(throws([&] { f.locate_moe_layer(1); }, MUMMU_ERR_RANGE, "layer 1"), "layer outside the file");
    }
    ::unlink(path.c_str());
    // refusals: magic, truncation, a bank with swapped dims
    {
        GgufBytes w = toy_gguf(r, g, u, d);
        std::string p2 = w.write("bad.gguf");
        FILE *fp = std::fopen(p2.c_str(), "r+b");
        if (fp) {
            std::fwrite("FUGG", 1, 4, fp);
            std::fclose(fp);
        }
        EXPECT(throws([&] { mummu::GgufFile::open(p2); }, MUMMU_ERR_GGUF, "not a GGUF file"), "bad magic");
        ::unlink(p2.c_str());
        EXPECT(throws([&] { mummu::GgufFile::open(p2); }, MUMMU_ERR_IO, "cannot open"), "missing file");
        GgufBytes sw;
        sw.kvs = w.kvs;
        sw.n_kv = w.n_kv;
        sw.tensor("blk.0.ffn_gate_inp.weight", {H, E}, 0, r.data(), r.size() * 4);
        sw.tensor("blk.0.ffn_gate_exps.weight", {I, H, E}, 0, g.data(), g.size() * 4);
        sw.tensor("blk.0.ffn_up_exps.weight", {H, I, E}, 0, u.data(), u.size() * 4);
        sw.tensor("blk.0.ffn_down_exps.weight", {I, H, E}, 0, d.data(), d.size() * 4);
        const std::string p3 = sw.write("swapped.gguf");
        mummu::GgufFile f = mummu::GgufFile::open(p3);
        EXPECT(throws([&] { f.locate_moe_layer(0); }, MUMMU_ERR_SHAPE, "ffn_gate_exps.weight: dim 0"), "swapped bank dims");
        ::unlink(p3.c_str());
    }
}

int main(int argc, char **argv) {
    const bool no_gpu = argc > 1 && std::string(argv[1]) == "--no-gpu";
    mummu::SparseMoeConfig cfg;
    cfg.hidden_size = H;
    cfg.expert_intermediate_size = I;
    cfg.num_experts = E;
    cfg.num_experts_per_tok = K;
    cfg.max_tokens = 8;

    // SparseMoeConfig::init refuses a block that is not a mixture (nn/moe.rs:62-76)
    {
        mummu::SparseMoeConfig bad = cfg;
        bad.num_experts = 1;
        EXPECT(throws([&] { mummu::SparseMoe m(bad); }, MUMMU_ERR_CONFIG, "experts"), "num_experts = 1 must be refused");
        bad = cfg;
        bad.num_experts_per_tok = E + 1;
        EXPECT(throws([&] { mummu::SparseMoe m(bad); }, MUMMU_ERR_CONFIG, "num_experts_per_tok"), "top_k > E must be refused");
        bad = cfg;
        bad.hidden_size = 0;
        EXPECT(throws([&] { mummu::SparseMoe m(bad); }, MUMMU_ERR_CONFIG, "hidden"), "zero hidden size must be refused");
    }
    {
        const std::vector<float> r = router_eh(), g = sin_fill(0.1f, E * I * H), u = sin_fill(1.7f, E * I * H),
                                 d = sin_fill(3.3f, E * H * I);
        gguf_host_checks(r, g, u, d);
    }
    // OlmoeConfig::from_json_bytes: fields, default, refusals (models/olmoe.rs:52-226)
    {
        const std::string ok = R"({"vocab_size": 50304, "hidden_size": 2048, "intermediate_size": 1024, "num_hidden_layers": 16,
            "num_attention_heads": 16, "num_key_value_heads": 16, "num_experts": 64, "num_experts_per_tok": 8,
            "rms_norm_eps": 1e-05, "rope_theta": 10000.0})";
        const mummu::SparseMoeConfig c = mummu::olmoe_config_from_json(ok);
        EXPECT(c.hidden_size == 2048 && c.expert_intermediate_size == 1024 && c.num_experts == 64 && c.num_experts_per_tok == 8 &&
                   c.num_layers == 16 && !c.norm_topk_prob,
               "config.json fields, norm_topk_prob defaults to false");
        std::string one = ok;
        one.replace(one.find("\"num_experts\": 64"), 17, "\"num_experts\": 1 ");
        EXPECT(throws([&] { mummu::olmoe_config_from_json(one); }, MUMMU_ERR_CONFIG, "num_experts (1) must be >= 2"), "one expert is refused");
        EXPECT(throws([&] { mummu::olmoe_config_from_json("{\"hidden_size\": 4"); }, MUMMU_ERR_CONFIG, "config.json"), "broken JSON is refused");
        EXPECT(throws([&] { mummu::Checkpoint::open("/nonexistent-dir"); }, MUMMU_ERR_IO, "neither"), "a directory without a checkpoint");
    }
    if (no_gpu) {
        std::printf(failures ? "host mirror: %d failure(s)\n" : "host mirror (no gpu): ok\n", failures);
        return failures ? 1 : 0;
    }

    const std::vector<float> r = router_eh(), g = sin_fill(0.1f, E * I * H), u = sin_fill(1.7f, E * I * H),
                             d = sin_fill(3.3f, E * H * I);
    mummu::SparseMoe moe(cfg);
    moe.load_layer(0, {r.data(), MUMMU_F32}, {g.data(), MUMMU_F32}, {u.data(), MUMMU_F32}, {d.data(), MUMMU_F32});
    EXPECT(moe.resident_bytes() == (uint64_t)4 * (E * H + 3 * E * I * H), "resident bytes");

    for (int t : {5, 1})
        for (bool norm : {false, true})
            for (int k : {K, E}) {
                const std::vector<float> x = input(t, 0.0f);
                const std::vector<float> got = moe.forward(x, k, norm), want = reference(r, g, u, d, x, t, k, norm);
                float worst = 0.0f;
                for (size_t i = 0; i < got.size(); i++) worst = std::fmax(worst, std::fabs(got[i] - want[i]));
                EXPECT(worst <= 1e-5f, "forward vs hand-rolled reference (1e-5 absolute, nn/moe.rs:2197)");
                // routed == fused, bit for bit; every token spends top_k hits
                (void)moe.take_hits();
                const mummu::Routing routing = moe.route(x, k, norm);
                const std::vector<float> routed = moe.run_local(x, routing);
                EXPECT(std::memcmp(routed.data(), got.data(), got.size() * 4) == 0, "run_local(route(x)) == forward(x)");
                size_t served = 0;
                for (const auto &pe : routing.per_expert) {
                    served += pe.first.size();
                    for (size_t i = 1; i < pe.first.size(); i++) EXPECT(pe.first[i - 1] < pe.first[i], "rows ascend per expert");
                }
                EXPECT(served == (size_t)(t * k), "every token is served top_k times");
                uint64_t hits = 0;
                for (uint64_t hh : moe.take_hits()) hits += hh;
                EXPECT(hits == (uint64_t)(t * k), "hit counters count the rows run_local served (route alone serves none)");
            }

    // the same block read back from a model file gives the same bits
    {
        const std::string path = toy_gguf(r, g, u, d).write("load.gguf");
        {
            mummu::GgufFile f = mummu::GgufFile::open(path);
            mummu::SparseMoe from_file = mummu::SparseMoe::from_gguf(f, 0, -1, 8);
            EXPECT(from_file.resident_bytes() == moe.resident_bytes(), "resident bytes after load_gguf");
            const std::vector<float> x = input(5, 2.0f);
            const std::vector<float> a = from_file.forward(x, K, true), b = moe.forward(x, K, true);
            EXPECT(std::memcmp(a.data(), b.data(), a.size() * 4) == 0, "from_gguf(file) == load_layer(bytes)");
        }
        ::unlink(path.c_str());
    }

    // zero in, zero out (nn/moe.rs:2340-2352)
    {
        const std::vector<float> z((size_t)(3 * H), 0.0f);
        for (float v : moe.forward(z, K, false)) EXPECT(v == 0.0f, "zero input gives zero output");
    }
    // contract violations are loud (nn/moe.rs:119-130)
    {
        const std::vector<float> x = input(2, 0.0f);
        EXPECT(throws([&] { moe.forward(x, 0, false); }, MUMMU_ERR_TOPK, "top_k"), "top_k = 0");
        EXPECT(throws([&] { moe.forward(x, E + 1, false); }, MUMMU_ERR_TOPK, "top_k"), "top_k > E");
        EXPECT(throws([&] { moe.forward(std::vector<float>(7), K, false); }, MUMMU_ERR_SHAPE, "hidden"), "ragged input");
        EXPECT(throws([&] { moe.forward(x, K, false, 1); }, MUMMU_ERR_RANGE, "layer"), "layer out of range");
    }
    // ExpertExec seam: one expert alone equals a top-1 routing to it with weight 1
    {
        mummu::HipExpert ex(moe, 0, 2);
        const std::vector<float> x = input(3, 1.0f);
        const std::vector<float> y = ex.run(x.data(), 3, H);
        mummu::RoutedExperts re(moe);
        const std::vector<float> y2 = re.apply_routing(0, {2, 2, 2}, {1.0f, 1.0f, 1.0f}, x, 3, 1);
        EXPECT(std::memcmp(y.data(), y2.data(), y.size() * 4) == 0, "ExpertExec::run == apply_routing(top-1, weight 1)");
        // the rest of the trait: pinned to device 0, always staged, gate energy = sum_i silu(x . gate_i)^2 >= 0
        const std::vector<float> en = ex.gate_energy(x.data(), 3, H);
        EXPECT(en.size() == 3 && std::isfinite(en[0]) && en[0] > 0.0f && en[1] > 0.0f && en[2] > 0.0f, "gate_energy finite and positive");
        const std::vector<float> en1 = ex.gate_energy(x.data() + H, 1, H);
        EXPECT(std::memcmp(&en1[0], &en[1], 4) == 0, "gate_energy of a row does not depend on the rows beside it");
        ex.stage(0);
        ex.evict();
        ex.disable_native();
        EXPECT(ex.tier().device == 0 && ex.is_staged(), "tier / is_staged");
        EXPECT(throws([&] { re.apply_routing(0, {2, 9, 2}, {1.0f, 1.0f, 1.0f}, x, 3, 1); }, MUMMU_ERR_RANGE, "expert"), "bad expert id");
    }
    // the packed GEMV op: a weight whose every code is -8 with unit scales against a row of ones gives -8 K
    {
        const int PK = 64, PN = 64;
        std::vector<uint32_t> words((size_t)PK * PN / 8, 0x88888888u);
        std::vector<float> scales((size_t)PK * PN / 32, 1.0f);
        mummu::PackedWeight pw(words, scales, PK, PN);
        const std::vector<float> y = pw.gemv(std::vector<float>(PK, 1.0f));
        bool all = y.size() == (size_t)PN;
        for (float v : y) all = all && v == -8.0f * PK;
        EXPECT(all, "q4s_gemv decodes two's complement nibbles");
        EXPECT(pw.resident_bytes() == (uint64_t)PK * PN / 2 + (uint64_t)PK * PN / 8, "packed weight bytes");
        EXPECT(throws([&] { pw.gemv(std::vector<float>(PK + 1, 0.0f)); }, MUMMU_ERR_SHAPE, "rows"), "ragged packed input");
    }
    // route known answers (experts.rs:1365-1388)
    {
        const std::vector<float> logits = {0.0f, 3.0f, 1.0f, 2.5f, -2.0f, 2.0f, 0.5f, 2.9f};
        auto rw = mummu::route(moe, logits, 1, 8, 3);
        EXPECT(rw.first == (std::vector<int32_t>{1, 7, 3}), "route ids [1,7,3]");
        double sum = 0.0, den = std::exp(3.0) + std::exp(2.9) + std::exp(2.5);
        for (int s = 0; s < 3; s++) {
            sum += rw.second[(size_t)s];
            EXPECT(std::fabs(rw.second[(size_t)s] - std::exp((double)logits[(size_t)rw.first[(size_t)s]]) / den) < 1e-6, "route weights");
        }
        EXPECT(std::fabs(sum - 1.0) < 1e-6, "weights sum to 1");
        auto tie = mummu::route(moe, {1.0f, 1.0f, 1.0f, 1.0f}, 1, 4, 3);
        EXPECT(tie.first == (std::vector<int32_t>{0, 1, 2}), "ties keep the lower id");
        auto tie2 = mummu::route(moe, {1.0f, 0.0f, 2.0f, 1.0f}, 1, 4, 2);
        EXPECT(tie2.first == (std::vector<int32_t>{2, 0}), "[1,0,2,1] k=2 -> [2,0]");
        const float nan = std::nanf("");
        EXPECT(throws([&] { mummu::route(moe, {0.0f, nan, 1.0f}, 1, 3, 1); }, MUMMU_ERR_NONFINITE, "finite"), "NaN logit refused");
        EXPECT(throws([&] { mummu::route(moe, {0.0f, 1.0f}, 1, 2, 3); }, MUMMU_ERR_TOPK, "top-3"), "k > E refused");
    }
    std::printf(failures ? "host mirror: %d failure(s)\n" : "host mirror: ok\n", failures);
    return failures ? 1 : 0;
}
