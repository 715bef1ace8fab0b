// C ABI of the sparse MoE block (include/mummu_moe.h): handle, weight residency, workspace,
// and the launch sequences.  Host logic only; the arithmetic lives in the kernel files.
#include "../../include/mummu_moe.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cstdlib>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "device_utils.h"
#include "kernels.h"

using namespace mummu;

namespace {

thread_local std::string g_error;  // failures of calls that have no handle

enum KernelSlot { K_ROUTER, K_ROUTER_LOGITS, K_ROUTE_TOPK, K_QUANTIZE, K_GATE_UP, K_DOWN_COMBINE, K_DOWN, K_COMBINE, K_RMSNORM,
                  K_DISPATCH, K_GEMM_GATE_UP, K_GEMM_DOWN, K_SHARED, K_DECODE_LAYER, K_SLOTS };
const char *const kSlotNames[K_SLOTS] = {"router", "router_logits", "route_topk", "quantize", "gate_up", "down_combine",
                                         "down", "combine", "rmsnorm", "dispatch", "gemm_gate_up", "gemm_down", "shared_expert",
                                         "decode_layer"};

struct Layer {
    void *router = nullptr;
    int router_type = 0;
    uint8_t *gate = nullptr, *up = nullptr, *down = nullptr;
    int gate_type = 0, up_type = 0, down_type = 0;
    float *gamma = nullptr;
    unsigned long long *hits = nullptr;
    size_t bytes = 0;
    bool loaded = false;
    bool q8_half_ok = false;     // all three banks Q8_0 and every |d| * 128 a finite half: the f16 kernel may take them
    // optional shared expert (always active) and its per-token sigmoid gate vector
    uint8_t *sh_gate = nullptr, *sh_up = nullptr, *sh_down = nullptr;
    int sh_gate_type = 0, sh_up_type = 0, sh_down_type = 0, sh_inter = 0;
    void *sh_gatevec = nullptr;  // [hidden], router-type floats; null: the shared expert is added ungated
    int sh_gatevec_type = 0;
    size_t sh_bytes = 0;
    bool sh_loaded = false;
};

struct TimedLaunch {
    hipEvent_t start, stop;
    int slot;
};

// What mummu_graph_end hands out: the executable graph and the handle generation it was captured under.
struct CapturedGraph {
    hipGraphExec_t exec;
    uint64_t generation;
};

}  // namespace

namespace mummu {
thread_local LaunchTiming g_launch_timing;
}

// Scratch of the entry point that allocates nothing (mummu_moe_forward_device_noalloc): what its three kernels hand to one
// another lives here instead of in hipMalloc'ed workspace.  Every GPU holds its own copy until the process ends.  In host
// code this name is only a stand-in for the symbol: the address kernels are given comes from hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[MUMMU_NOALLOC_SCRATCH_BYTES];

struct mummu_moe {
    mummu_moe_config cfg{};
    std::vector<Layer> layers;
    hipStream_t stream = nullptr;
    // pinned host staging for the host-pointer entry points: [input | output | flags]; small calls go through
    // it with asynchronous copies and one synchronisation
    uint8_t *pin = nullptr;
    std::mutex mu;
    mutable std::string err;

    // workspace (device)
    int64_t ws_tokens = 0, ws_assign = 0;
    int ws_experts = 0;
    float *logits = nullptr, *weights = nullptr, *act = nullptr, *y = nullptr;
    int32_t *ids = nullptr, *flags = nullptr;
    float *xin = nullptr, *xout = nullptr, *h2 = nullptr, *resid[2] = {nullptr, nullptr};
    QAct xq, actq;               // 16-bit activations: tokens x hidden, pairs x inter
    // dispatch-sorted layout of the batched path
    int32_t *offsets = nullptr, *sorted = nullptr, *inv = nullptr, *tiles = nullptr, *n_tiles = nullptr, *disp_scratch = nullptr;
    void *act16 = nullptr;       // f16 [pairs, inter]
    int max_tiles = 0;
    // batches at least this large take dispatch + grouped GEMM (measured crossovers on the OLMoE shape:
    // the 16-bit float decode kernels lose from 7 tokens on, the f32 ones from 10, the integer ones from 19)
    int gemm_min_f16 = 7, gemm_min_quant = 19, gemm_min_f32 = 10;
    int gemm_min_q4k = 18;   // Q4_K banks on the f16 units (17 tokens: 88.8 us either way; 18: 89.1 against 92.6 us)
    int gemm_q4k_f16 = 1;        // Q4_K banks of the batched path on the f16 units (0: the int8 form)
    int gemm_q8_f16 = 0;         // 1: Q8_0 banks of the batched path through the f16 kernel (x and activations as halfs)
    int gemm_tile_rows = 0;          // 0: chosen per batch; else forced (f16-unit Q4_K kernels)
    // shared-expert workspace: tokens x widest shared inter, tokens x hidden, tokens
    int sh_inter_max = 0;
    int64_t sh_ws_tokens = 0;
    float *sh_act = nullptr, *sh_y = nullptr;
    QAct sh_actq;
    void *sh_act16 = nullptr;                                   // f16 [tokens, shared inter]: batched path, F16 / BF16 banks
    int32_t *sh_sorted = nullptr, *sh_tiles = nullptr, *sh_ntiles = nullptr;  // its one-expert work list
    int sh_max_tiles = 0;

    // router exchange of the two-launch decode form (gate_up_fused_kernel): the per-XCD logit table, its epoch counter
    // and the count of workgroups that gave up waiting; xcd_round_robin says the device deals workgroups to 8 XCDs by
    // linear id modulo 8, which is what makes the exchange worth using
    void *xslots = nullptr;
    unsigned long long *xstate = nullptr;  // [0] epoch, [1] fallbacks
    bool xcd_round_robin = false;
    int router_exchange = 1;
    unsigned spin_ticks = 5000;
    unsigned long long fallbacks_seen = 0;   // the fallback counter at mummu_moe_check's last look
    // the one-launch decode form (decode_layer_kernel): the table its workgroups pass the experts' hidden rows through,
    // and a counter that tells launches apart which read the same epoch (the nodes of one captured graph)
    void *aslots = nullptr;
    int layer_fusion = 1;      // 0: never the one-launch form; 1: where its sum can be left to the next step; 2: wherever it serves
    int early_ids = 1;         // the fused decode launches start their rows on the eight largest logits and confirm them (MUMMU_EARLY_IDS=0: route first)
    int warm_next = 1;         // the one-launch decode form reads the next layer's router ahead at its end (MUMMU_WARM_NEXT=0: not)
    int tile_order = -1;       // decode launches of several tokens fetch a shared expert's rows once: -1 from six tokens on, 0 never, 1 from two (mummu_moe_set_tile_order)
    unsigned launch_salt = 0;
    // The weighted sum over a token's eight slots can be left to the launch of the NEXT device-pointer call (deferred_combine,
    // off by default), whose otherwise idle waves do it: the one-launch form then costs one launch per step.  The per-slot
    // rows and the routing of consecutive steps alternate between two sets of buffers ([0] = y, ids, weights above);
    // `pending` is the step whose sum has not been enqueued yet.
    int deferred_combine = 0;
    float *y_alt = nullptr, *weights_alt = nullptr;
    int32_t *ids_alt = nullptr;
    int decode_buf = 0;    // the set the next deferred step writes
    int routing_buf = 0;   // the set that holds the last call's routing
    struct {
        bool active = false;
        int buf = 0, k = 0;
        int64_t n = 0;
        const float *residual = nullptr;
        float *out = nullptr;
        hipStream_t stream = nullptr;
    } pending;
    // bumped whenever a device buffer a captured graph may point into is freed (workspace regrown, a layer's or
    // a shared expert's weights replaced); a graph remembers the value it was captured under
    uint64_t generation = 0;

    hipEvent_t t0 = nullptr, t1 = nullptr;
    bool timing = false;
    std::vector<TimedLaunch> timed;
    std::vector<hipEvent_t> event_pool;
};

namespace {

int fail(mummu_moe *h, int code, const std::string &msg) {
    if (h) h->err = msg;
    else g_error = msg;
    return code;
}

#define HIPCHK(h, call)                                                                                    \
    do {                                                                                                   \
        hipError_t e_ = (call);                                                                            \
        if (e_ != hipSuccess)                                                                              \
            return fail(h, MUMMU_ERR_DEVICE, std::string(#call) + ": " + hipGetErrorString(e_));            \
    } while (0)

int flush_pending(mummu_moe *h);

// Takes the handle's lock and, first of all, enqueues the weighted sum a deferred decode step may have left pending
// (see mummu_moe_set_deferred_combine): every entry point but the one that continues such a chain starts with this.
struct Entry {
    std::lock_guard<std::mutex> lock;
    int rc;
    explicit Entry(mummu_moe *h) : lock(h->mu), rc(flush_pending(h)) {}
};

// The device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(mummu_moe *h, unsigned char **out) {
    int dev = -1;
    HIPCHK(h, hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(h, MUMMU_ERR_DEVICE, "device index " + std::to_string(dev) + " out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        HIPCHK(h, hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(h, MUMMU_ERR_DEVICE, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[dev] = (unsigned char *)p;
    }
    *out = g_scratch_ptr[dev];
    return MUMMU_OK;
}

bool bank_type_ok(int t) { return block_elems(t) > 0; }  // F32, F16, BF16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K
bool router_type_ok(int t) { return t == T_F32 || t == T_F16 || t == T_BF16; }
size_t row_bytes_of(int t, int in_dim) { return (size_t)(in_dim / block_elems(t)) * (size_t)block_bytes(t); }

void free_ws(mummu_moe *h) {
    h->generation++;
    void *ptrs[] = {h->logits, h->weights, h->act, h->y, h->ids, h->xin, h->xout, h->h2, h->resid[0], h->resid[1],
                    h->xq.hi, h->xq.lo, h->xq.scale, h->xq.sum, h->actq.hi, h->actq.lo, h->actq.scale, h->actq.sum,
                    h->offsets, h->sorted, h->inv, h->tiles, h->n_tiles, h->act16, h->disp_scratch, h->y_alt, h->weights_alt, h->ids_alt};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    h->logits = h->weights = h->act = h->y = h->xin = h->xout = h->h2 = h->resid[0] = h->resid[1] = nullptr;
    h->ids = nullptr;
    h->y_alt = h->weights_alt = nullptr;
    h->ids_alt = nullptr;
    h->decode_buf = h->routing_buf = 0;
    h->xq = QAct();
    h->actq = QAct();
    h->offsets = h->sorted = h->inv = h->tiles = h->n_tiles = h->disp_scratch = nullptr;
    h->act16 = nullptr;
    h->ws_tokens = h->ws_assign = 0;
    h->ws_experts = 0;
    void *sh[] = {h->sh_act, h->sh_y, h->sh_actq.hi, h->sh_actq.lo, h->sh_actq.scale, h->sh_actq.sum,
                  h->sh_act16, h->sh_sorted, h->sh_tiles, h->sh_ntiles};
    for (void *p : sh)
        if (p) (void)hipFree(p);
    h->sh_act = h->sh_y = nullptr;
    h->sh_actq = QAct();
    h->sh_act16 = nullptr;
    h->sh_sorted = h->sh_tiles = h->sh_ntiles = nullptr;
    h->sh_ws_tokens = 0;
}

// The shared expert's own buffers, sized for the main workspace's token count.
int ensure_shared_ws(mummu_moe *h) {
    if (h->sh_inter_max == 0 || h->sh_ws_tokens >= h->ws_tokens) return MUMMU_OK;
    HIPCHK(h, hipDeviceSynchronize());
    h->generation++;
    void *sh[] = {h->sh_act, h->sh_y, h->sh_actq.hi, h->sh_actq.lo, h->sh_actq.scale, h->sh_actq.sum,
                  h->sh_act16, h->sh_sorted, h->sh_tiles, h->sh_ntiles};
    for (void *p : sh)
        if (p) (void)hipFree(p);
    h->sh_act = h->sh_y = nullptr;
    h->sh_actq = QAct();
    h->sh_act16 = nullptr;
    h->sh_sorted = h->sh_tiles = h->sh_ntiles = nullptr;
    const size_t nt = (size_t)h->ws_tokens, H = (size_t)h->cfg.hidden_size, I = (size_t)h->sh_inter_max;
    const size_t ae = nt * ((I + 15) / 16 * 16);
    HIPCHK(h, hipMalloc(&h->sh_act, sizeof(float) * nt * I));
    HIPCHK(h, hipMalloc(&h->sh_y, sizeof(float) * nt * H));
    HIPCHK(h, hipMalloc(&h->sh_actq.hi, ae));
    HIPCHK(h, hipMalloc(&h->sh_actq.lo, ae));
    HIPCHK(h, hipMalloc(&h->sh_actq.scale, sizeof(float) * (ae / 16)));
    HIPCHK(h, hipMalloc(&h->sh_actq.sum, sizeof(int32_t) * (ae / 16)));
    HIPCHK(h, hipMalloc(&h->sh_act16, 2 * nt * I));

    h->sh_max_tiles = (int)((nt + 31) / 32) + 1;
    HIPCHK(h, hipMalloc(&h->sh_sorted, sizeof(int32_t) * nt));
    HIPCHK(h, hipMalloc(&h->sh_tiles, sizeof(int32_t) * 3 * (size_t)h->sh_max_tiles));
    HIPCHK(h, hipMalloc(&h->sh_ntiles, sizeof(int32_t)));
    h->sh_ws_tokens = h->ws_tokens;
    return MUMMU_OK;
}

// Grow the workspace to hold n tokens and n_assign (token, expert) pairs.  Host entry points
// only: synchronises and reallocates.
int ensure_ws(mummu_moe *h, int64_t n, int64_t n_assign, int n_experts) {
    if (n_experts < h->cfg.num_experts) n_experts = h->cfg.num_experts;
    if (n <= h->ws_tokens && n_assign <= h->ws_assign && n_experts <= h->ws_experts) return MUMMU_OK;
    {
        const int rc = flush_pending(h);
        if (rc) return rc;
    }
    HIPCHK(h, hipDeviceSynchronize());
    int64_t nt = n > h->ws_tokens ? n : h->ws_tokens;
    int64_t na = n_assign > h->ws_assign ? n_assign : h->ws_assign;
    if (n_experts < h->ws_experts) n_experts = h->ws_experts;
    free_ws(h);
    const size_t H = (size_t)h->cfg.hidden_size, I = (size_t)h->cfg.expert_intermediate_size;
    const size_t E = (size_t)n_experts;
    HIPCHK(h, hipMalloc(&h->logits, sizeof(float) * (size_t)nt * E));
    HIPCHK(h, hipMalloc(&h->ids, sizeof(int32_t) * (size_t)na));
    HIPCHK(h, hipMalloc(&h->weights, sizeof(float) * (size_t)na));
    HIPCHK(h, hipMalloc(&h->act, sizeof(float) * (size_t)na * I));
    HIPCHK(h, hipMalloc(&h->y, sizeof(float) * (size_t)na * H));
    HIPCHK(h, hipMalloc(&h->xin, sizeof(float) * (size_t)nt * H));
    HIPCHK(h, hipMalloc(&h->xout, sizeof(float) * (size_t)nt * H));
    HIPCHK(h, hipMalloc(&h->h2, sizeof(float) * (size_t)nt * H));
    HIPCHK(h, hipMalloc(&h->resid[0], sizeof(float) * (size_t)nt * H));
    HIPCHK(h, hipMalloc(&h->resid[1], sizeof(float) * (size_t)nt * H));
    // quantized activations (element counts rounded up to whole 16-element blocks)
    const size_t xe = (size_t)nt * ((H + 15) / 16 * 16), ae = (size_t)na * ((I + 15) / 16 * 16);
    HIPCHK(h, hipMalloc(&h->xq.hi, xe));
    HIPCHK(h, hipMalloc(&h->xq.lo, xe));
    HIPCHK(h, hipMalloc(&h->xq.scale, sizeof(float) * (xe / 16)));
    HIPCHK(h, hipMalloc(&h->xq.sum, sizeof(int32_t) * (xe / 16)));
    HIPCHK(h, hipMalloc(&h->actq.hi, ae));
    HIPCHK(h, hipMalloc(&h->actq.lo, ae));
    HIPCHK(h, hipMalloc(&h->actq.scale, sizeof(float) * (ae / 16)));
    HIPCHK(h, hipMalloc(&h->actq.sum, sizeof(int32_t) * (ae / 16)));
    h->max_tiles = n_experts + (int)((na + 15) / 16) + 1;   // (the smallest tiles have 16 rows)
    HIPCHK(h, hipMalloc(&h->offsets, sizeof(int32_t) * (size_t)(n_experts + 1)));
    HIPCHK(h, hipMalloc(&h->sorted, sizeof(int32_t) * (size_t)na));
    HIPCHK(h, hipMalloc(&h->inv, sizeof(int32_t) * (size_t)na));
    HIPCHK(h, hipMalloc(&h->tiles, sizeof(int32_t) * 3 * (size_t)h->max_tiles));
    HIPCHK(h, hipMalloc(&h->n_tiles, sizeof(int32_t)));
    HIPCHK(h, hipMalloc(&h->disp_scratch, sizeof(int32_t) * dispatch_scratch_ints((int)na, n_experts)));
    HIPCHK(h, hipMalloc(&h->act16, 2 * (size_t)na * I));
    {
        // the second set of the deferred sums' buffers: decode steps only (at most kExchangeTokens tokens)
        const size_t na8 = (size_t)std::min<int64_t>(na, (int64_t)kExchangeTokens * 8);
        HIPCHK(h, hipMalloc(&h->y_alt, sizeof(float) * na8 * H));
        HIPCHK(h, hipMalloc(&h->ids_alt, sizeof(int32_t) * na8));
        HIPCHK(h, hipMalloc(&h->weights_alt, sizeof(float) * na8));
    }
    h->ws_tokens = nt;
    h->ws_assign = na;
    h->ws_experts = n_experts;
    return ensure_shared_ws(h);
}

// Device error flags back to idle.
constexpr int kFlagWords = 4;

int reset_flags(mummu_moe *h) {
    const int32_t init[kFlagWords] = {0, INT_MAX, 0, 0};
    HIPCHK(h, hipMemcpy(h->flags, init, sizeof(init), hipMemcpyHostToDevice));
    return MUMMU_OK;
}

int flags_to_status(mummu_moe *h, const int32_t *f);

constexpr unsigned long long kFallbacksBeforeGivingUp = 64;

// Synchronise and translate the device error flags.
int check_flags(mummu_moe *h, hipStream_t s) {
    HIPCHK(h, hipStreamSynchronize(s));
    int32_t f[4];
    HIPCHK(h, hipMemcpy(f, h->flags, sizeof(f), hipMemcpyDeviceToHost));
    if (h->router_exchange == 1 && h->xstate != nullptr) {
        // Workgroups of the fused decode forms that gave up waiting for the others since the last look: each of them sat
        // out its bound (spin_ticks, tens of microseconds against a step of 15) before it computed what it missed - the
        // device is shared, or it does not place workgroups the way the probe saw.  The result is right either way, but
        // the three-launch form is the faster one then: fall back to it for the rest of this handle's life.  (A caller
        // that set the form explicitly - mummu_moe_set_router_exchange with 0 or 2 - keeps what it asked for.)
        unsigned long long fb = 0;
        HIPCHK(h, hipMemcpy(&fb, h->xstate + 1, sizeof(fb), hipMemcpyDeviceToHost));
        if (fb - h->fallbacks_seen >= kFallbacksBeforeGivingUp) h->router_exchange = 0;
        h->fallbacks_seen = fb;
    }
    return flags_to_status(h, f);
}

int flags_to_status(mummu_moe *h, const int32_t *f) {
    if (f[FLAG_NONFINITE] == 0 && f[FLAG_BAD_ID] == 0) return MUMMU_OK;
    int rc = reset_flags(h);
    if (rc != MUMMU_OK) return rc;
    if (f[FLAG_NONFINITE]) {
        const int E = h->cfg.num_experts;
        char buf[160];
        snprintf(buf, sizeof(buf), "router logit for token %d expert %d is not finite", f[FLAG_NONFINITE_INDEX] / E,
                 f[FLAG_NONFINITE_INDEX] % E);
        return fail(h, MUMMU_ERR_NONFINITE, buf);
    }
    return fail(h, MUMMU_ERR_RANGE, "a routed expert id is out of range");
}

// Host-pointer calls of up to kPinIO bytes each way: the input is staged through pinned memory (the
// copy is then truly asynchronous), and the output and the error flags come back with one
// synchronisation instead of one per copy.  Larger calls copy straight from / to the caller's memory.
constexpr size_t kPinIO = 256 * 1024;

// The routing of n*k pairs back to the caller (ids, weights; logits too when asked for) under one
// synchronisation, with the error flags.
int download_routing(mummu_moe *h, int32_t *ids, float *weights, size_t pairs, float *logits, size_t n_logits, hipStream_t s);

// (pin_offset: where in the input half this upload is staged - a call with two inputs gives each its own place)
int upload_rows(mummu_moe *h, float *dev, const float *host, size_t bytes, hipStream_t s, size_t pin_offset = 0) {
    if (h->pin && pin_offset + bytes <= kPinIO) {
        memcpy(h->pin + pin_offset, host, bytes);
        HIPCHK(h, hipMemcpyAsync(dev, h->pin + pin_offset, bytes, hipMemcpyHostToDevice, s));
    } else {
        HIPCHK(h, hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, s));
    }
    return MUMMU_OK;
}

// Wait for the stream, report what the device flagged, hand the result rows to the caller.
int download_rows(mummu_moe *h, float *host, const float *dev, size_t bytes, hipStream_t s, bool with_flags) {
    if (h->pin && bytes <= kPinIO) {
        int32_t *pf = (int32_t *)(h->pin + 2 * kPinIO);
        if (with_flags) HIPCHK(h, hipMemcpyAsync(pf, h->flags, sizeof(int32_t) * kFlagWords, hipMemcpyDeviceToHost, s));
        HIPCHK(h, hipMemcpyAsync(h->pin + kPinIO, dev, bytes, hipMemcpyDeviceToHost, s));
        HIPCHK(h, hipStreamSynchronize(s));
        if (with_flags) {
            const int rc = flags_to_status(h, pf);
            if (rc) return rc;
        }
        memcpy(host, h->pin + kPinIO, bytes);
        return MUMMU_OK;
    }
    if (with_flags) {
        const int rc = check_flags(h, s);
        if (rc) return rc;
    } else {
        HIPCHK(h, hipStreamSynchronize(s));
    }
    HIPCHK(h, hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    return MUMMU_OK;
}

int download_routing(mummu_moe *h, int32_t *ids, float *weights, size_t pairs, float *logits, size_t n_logits, hipStream_t s) {
    const size_t ib = sizeof(int32_t) * pairs, wb = sizeof(float) * pairs, lb = logits ? sizeof(float) * n_logits : 0;
    if (h->pin && ib + wb + lb <= kPinIO) {
        uint8_t *p = h->pin + kPinIO;
        int32_t *pf = (int32_t *)(h->pin + 2 * kPinIO);
        HIPCHK(h, hipMemcpyAsync(pf, h->flags, sizeof(int32_t) * kFlagWords, hipMemcpyDeviceToHost, s));
        HIPCHK(h, hipMemcpyAsync(p, h->ids, ib, hipMemcpyDeviceToHost, s));
        HIPCHK(h, hipMemcpyAsync(p + ib, h->weights, wb, hipMemcpyDeviceToHost, s));
        if (lb) HIPCHK(h, hipMemcpyAsync(p + ib + wb, h->logits, lb, hipMemcpyDeviceToHost, s));
        HIPCHK(h, hipStreamSynchronize(s));
        const int rc = flags_to_status(h, pf);
        if (rc) return rc;
        memcpy(ids, p, ib);
        memcpy(weights, p + ib, wb);
        if (lb) memcpy(logits, p + ib + wb, lb);
        return MUMMU_OK;
    }
    const int rc = check_flags(h, s);
    if (rc) return rc;
    HIPCHK(h, hipMemcpy(ids, h->ids, ib, hipMemcpyDeviceToHost));
    HIPCHK(h, hipMemcpy(weights, h->weights, wb, hipMemcpyDeviceToHost));
    if (lb) HIPCHK(h, hipMemcpy(logits, h->logits, lb, hipMemcpyDeviceToHost));
    return MUMMU_OK;
}

// Per-kernel timing: binds a pair of pooled events to the one kernel the enclosed launcher
// dispatches (see launch_kernel).
struct ScopedTimer {
    bool armed = false;
    ScopedTimer(mummu_moe *h, hipStream_t, int slot) {
        if (!h->timing) return;
        hipEvent_t ev[2];
        for (auto &e : ev) {
            if (!h->event_pool.empty()) {
                e = h->event_pool.back();
                h->event_pool.pop_back();
            } else if (hipEventCreate(&e) != hipSuccess) {
                return;
            }
        }
        g_launch_timing.start = ev[0];
        g_launch_timing.stop = ev[1];
        armed = true;
        h->timed.push_back({ev[0], ev[1], slot});
    }
    ~ScopedTimer() {
        if (armed) g_launch_timing = LaunchTiming();
    }
};

#define LAUNCH(h, slot, s, call)                                                                 \
    do {                                                                                         \
        hipError_t e_;                                                                           \
        {                                                                                        \
            ScopedTimer timer_(h, s, slot);                                                      \
            e_ = (call);                                                                         \
        }                                                                                        \
        if (e_ != hipSuccess)                                                                    \
            return fail(h, MUMMU_ERR_DEVICE, std::string(#call) + ": " + hipGetErrorString(e_));  \
    } while (0)

ExpertBanks banks_of(const mummu_moe *h, const Layer &L) {
    ExpertBanks b;
    b.gate = L.gate;
    b.up = L.up;
    b.down = L.down;
    b.gate_type = L.gate_type;
    b.up_type = L.up_type;
    b.down_type = L.down_type;
    b.hidden = h->cfg.hidden_size;
    b.inter = h->cfg.expert_intermediate_size;
    b.n_experts = h->cfg.num_experts;
    b.q8_half_ok = L.q8_half_ok;
    b.tile_order_from = h->tile_order < 0 ? 6 : (h->tile_order == 0 ? 0x7fffffff : 2);
    b.early_ids = h->early_ids != 0;
    return b;
}

int check_layer(mummu_moe *h, int layer) {
    if (layer < 0 || layer >= (int)h->layers.size())
        return fail(h, MUMMU_ERR_RANGE, "layer " + std::to_string(layer) + " out of range (" + std::to_string(h->layers.size()) + ")");
    if (!h->layers[layer].loaded) return fail(h, MUMMU_ERR_NOT_LOADED, "layer " + std::to_string(layer) + " has no weights");
    return MUMMU_OK;
}

int check_topk(mummu_moe *h, int top_k, int n_experts) {
    if (top_k < 1 || top_k > n_experts)
        return fail(h, MUMMU_ERR_TOPK, "MoE forward: top_k (" + std::to_string(top_k) + ") must be in 1..=num_experts (" +
                                           std::to_string(n_experts) + ")");
    return MUMMU_OK;
}

// experts of an already-made routing: gate/up -> down -> combine.  x_quantized says h->xq
// already holds the 16-bit form of x (the fused router produced it).
// Smallest batch of this layer that takes the batched path (INT_MAX: never).
int batched_from(const mummu_moe *h, const Layer &L) {
    const ExpertBanks b = banks_of(h, L);
    if (!grouped_gemm_supported(b)) return 0x7fffffff;
    if (b.gate_type == T_F32) return h->gemm_min_f32;
    if (h->gemm_q4k_f16 && grouped_gemm_q4k_f16_down(b)) return h->gemm_min_q4k;
    return grouped_gemm_quantized(b) ? h->gemm_min_quant : h->gemm_min_f16;
}

// Q4_K banks on the f16 units (batched path): whether gate/up (hf) and down (hf_down) take that form for this batch,
// and where x goes as pairs of halfs: the (not yet written) buffer of the down product's output.
struct HalfPlan {
    bool hf = false, hf_down = false;
    HAct xh;
};

HalfPlan half_plan(const mummu_moe *h, const ExpertBanks &b, int64_t n, int k) {
    HalfPlan p;
    const size_t na = (size_t)(n * k);
    // (its kernels address the activation planes with 32-bit byte offsets)
    const bool small32 = na * (size_t)(b.hidden > b.inter ? b.hidden : b.inter) * 2 < (1ull << 32);
    p.hf = h->gemm_q4k_f16 && small32 && grouped_gemm_q4k_f16(b);
    p.hf_down = p.hf && grouped_gemm_q4k_f16_down(b);
    // x as pairs of halfs borrows h->y (the down product's output, written only after the gate/up launch has read x) and
    // the scale / sum arrays of the 16-bit form (unused on this path): run_experts keeps the order quantize -> gate/up ->
    // down on one stream, and nothing else may hold h->y across the gate/up launch
    if (p.hf) p.xh = HAct{(_Float16 *)h->y, (_Float16 *)h->y + (size_t)n * b.hidden, h->xq.scale, (float *)h->xq.sum};
    return p;
}

int run_experts(mummu_moe *h, const Layer &L, const float *x, bool x_quantized, int64_t n, int k, const float *residual,
                float *out, hipStream_t s, bool count_hits = false, bool xh_done = false) {
    ExpertBanks b = banks_of(h, L);
    const int na = (int)(n * k);
    if (n >= batched_from(h, L)) {
        // batched: sort the assignments by expert, then one grouped GEMM per projection
        // the 16-bit activation buffers, viewed in the batched path's 64-element-block layout
        const QAct64 xq64{h->xq.hi, h->xq.lo, h->xq.scale, (float *)h->xq.sum};
        const QAct64 actq64{h->actq.hi, h->actq.lo, h->actq.scale, (float *)h->actq.sum};
        // Q4_K banks on the f16 units: x as pairs of halfs in the (not yet written) buffer of the down product's
        // output, the activations between the two products in the f16 and f32 activation buffers
        const HalfPlan hp = half_plan(h, b, n, k);
        const bool hf = hp.hf, hf_down = hp.hf_down;
        // Q8_0 banks through the f16 kernel: x as halfs, like the f16 banks
        const bool q8h = h->gemm_q8_f16 && grouped_gemm_q8_f16(b);
        int tile_rows = hf_down ? grouped_gemm_tile_rows_q4k_f16(na, b.n_experts) : grouped_gemm_tile_rows(b, na, b.n_experts, q8h);
        if (hf_down && h->gemm_tile_rows != 0) tile_rows = h->gemm_tile_rows;
        // (the launches' grids cover the most tiles this batch can have, not the most the workspace holds)
        const int tiles_bound = std::min(h->max_tiles, b.n_experts + (na + tile_rows - 1) / tile_rows + 1);
        // (f16 / bf16 banks: x as halfs in the same buffer)
        const bool half_banks = b.gate_type == T_F16 || b.gate_type == T_BF16 || q8h;
        const HAct xh = hf ? hp.xh : (half_banks ? HAct{(_Float16 *)h->y, nullptr, nullptr, nullptr} : HAct());
        const HAct acth = hf_down ? HAct{(_Float16 *)h->act16, (_Float16 *)h->act, h->actq.scale, (float *)h->actq.sum} : HAct();
        if (hf && !xh_done) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows_h(x, (int)n, b.hidden, xh, s));
        else if (hf) {}   // (the router launch wrote them)
        else if (half_banks) LAUNCH(h, K_QUANTIZE, s, launch_convert_rows_f16(x, (int)n, b.hidden, xh.hi, s));
        else if (grouped_gemm_quantized(b)) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows64(x, (int)n, b.hidden, xq64, s));
        LAUNCH(h, K_DISPATCH, s,
               launch_dispatch(h->ids, na, b.n_experts, tile_rows, h->offsets, h->sorted, h->inv, h->tiles, h->n_tiles, h->disp_scratch,
                               count_hits ? L.hits : nullptr, h->flags, s));
        LAUNCH(h, K_GEMM_GATE_UP, s,
               launch_gemm_gate_up(b, x, xq64, xh, h->sorted, k, h->tiles, h->n_tiles, tiles_bound, tile_rows, h->act16, h->act, actq64,
                                   acth, s, q8h));
        LAUNCH(h, K_GEMM_DOWN, s,
               launch_gemm_down(b, h->act16, h->act, actq64, acth, na, h->tiles, h->n_tiles, tiles_bound, tile_rows, h->y, s, q8h));
        LAUNCH(h, K_COMBINE, s, launch_combine(h->y, h->ids, h->weights, h->inv, (int)n, k, b.hidden, residual, out, s));
        return MUMMU_OK;
    }
    if (is_quant_type(b.gate_type) && !x_quantized)
        LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows(x, (int)n, b.hidden, h->xq, s));
    LAUNCH(h, K_GATE_UP, s, launch_gate_up(b, x, h->xq, h->ids, na, k, -1, h->act, h->actq, h->flags, s));
    if (down_combine_supported(b, k)) {
        LAUNCH(h, K_DOWN_COMBINE, s, launch_down_combine(b, h->actq, h->ids, h->weights, (int)n, k, residual, out, s));
    } else {
        LAUNCH(h, K_DOWN, s, launch_down(b, h->act, h->actq, h->ids, na, k, -1, h->y, s));
        LAUNCH(h, K_COMBINE, s, launch_combine(h->y, h->ids, h->weights, nullptr, (int)n, k, b.hidden, residual, out, s));
    }
    return MUMMU_OK;
}

// The three-launch decode form (router logits + quantization, gate/up with the routing inside,
// down + combine): nothing but the first launch reads the float activations.
bool decode_three_launches(const mummu_moe *h, const Layer &L, int64_t n, int k) {
    const int E = h->cfg.num_experts, H = h->cfg.hidden_size;
    const ExpertBanks b = banks_of(h, L);
    const bool batched = n >= batched_from(h, L);
    const bool want_xq = is_quant_type(L.gate_type) && H % 64 == 0 && !batched;
    return !(n > 8 && router_fused_supported(E)) && want_xq && gate_up_routes_inline(b, k) && down_combine_supported(b, k);
}

// What the three-launch decode form keeps between its launches: the router's logits, the routing the gate/up kernel
// publishes, and the 16-bit activations of the block's input and of the experts' hidden rows.
struct DecodeScratch {
    float *logits;    // [n, E]
    int32_t *ids;     // [n, k]
    float *weights;   // [n, k]
    QAct xq, actq;    // [n, H] and [n*k, I rounded up to 16]
    void *xslots = nullptr;                  // router exchange table (router_exchange_bytes(E)), or null: three launches
    unsigned long long *xstate = nullptr;    // [0] its epoch, [1] its fallback counter
    void *aslots = nullptr;                  // hidden-row exchange table (layer_exchange_bytes()), or null: no one-launch form
    float *y = nullptr;                      // [n*k, H]: per-slot down sums of the one-launch form
};

// The two launches after the router's: gate/up with the routing inside, then down + combine.
int decode_tail(mummu_moe *h, const Layer &L, const DecodeScratch &ws, int n, int k, int norm, const float *residual, float *out,
                hipStream_t s) {
    const ExpertBanks b = banks_of(h, L);
    RouteInline route;
    route.logits = ws.logits;
    route.flavour = h->cfg.router_flavour;
    route.norm = norm;
    route.ids = ws.ids;
    route.weights = ws.weights;
    route.hits = L.hits;
    LAUNCH(h, K_GATE_UP, s, launch_gate_up_routed(b, ws.xq, route, n, k, ws.actq, h->flags, s));
    LAUNCH(h, K_DOWN_COMBINE, s, launch_down_combine(b, ws.actq, ws.ids, ws.weights, n, k, residual, out, s));
    return MUMMU_OK;
}

// The two sets of buffers consecutive deferred steps alternate between.
struct DecodeBuffers {
    float *y;
    int32_t *ids;
    float *weights;
};

DecodeBuffers decode_buffers(const mummu_moe *h, int buf) {
    return buf == 0 ? DecodeBuffers{h->y, h->ids, h->weights} : DecodeBuffers{h->y_alt, h->ids_alt, h->weights_alt};
}

// Enqueues the weighted sum a deferred step left pending (on the stream that step ran on) and moves the exchange's epoch on.
int flush_pending(mummu_moe *h) {
    if (!h->pending.active) return MUMMU_OK;
    h->pending.active = false;
    const DecodeBuffers pb = decode_buffers(h, h->pending.buf);
    hipStream_t s = h->pending.stream;
    LAUNCH(h, K_COMBINE, s,
           launch_combine(pb.y, pb.ids, pb.weights, nullptr, (int)h->pending.n, h->pending.k, h->cfg.hidden_size, h->pending.residual,
                          h->pending.out, s, h->xstate));
    return MUMMU_OK;
}

// What the fused decode launches are told about the router and the exchange.
RouterExchange router_exchange_of(mummu_moe *h, const Layer &L, const DecodeScratch &ws, const float *x, const float *norm_gamma,
                                  float *xnorm_out) {
    RouterExchange rx;
    rx.x = x;
    rx.w = L.router;
    rx.wtype = L.router_type;
    rx.gamma = norm_gamma;
    rx.eps = h->cfg.rms_norm_eps;
    rx.xnorm_out = xnorm_out;
    rx.slots = ws.xslots;
    rx.epoch = ws.xstate;
    rx.logits_out = ws.logits;
    rx.spin_ticks = h->spin_ticks;
    rx.fallbacks = ws.xstate + 1;
    rx.salt = ++h->launch_salt;
    if (L.sh_loaded) rx.xq_out = ws.xq;  // the shared expert's kernels multiply the same 16-bit rows
    return rx;
}

// The decode step as one expert launch (router + routing + gate/up + down, see decode_layer_kernel) followed by the
// weighted sum over each token's slots.  *done = false: not taken, nothing launched.
int decode_one_launch(mummu_moe *h, const Layer &L, const DecodeScratch &ws, const float *x, int n, int k, int norm,
                      const float *residual, float *out, hipStream_t s, const float *norm_gamma, float *xnorm_out, bool may_defer,
                      bool *done) {
    *done = false;
    if (!h->layer_fusion || !h->router_exchange || !h->xcd_round_robin || ws.xslots == nullptr || ws.xstate == nullptr ||
        ws.aslots == nullptr || ws.y == nullptr)
        return MUMMU_OK;
    if (n > 1 && h->router_exchange < 2) return MUMMU_OK;  // (like the two-launch form: every workgroup of every token repeats the waits)
    const ExpertBanks b = banks_of(h, L);
    LayerExchange lx;
    lx.act_slots = ws.aslots;
    lx.y = ws.y;
    lx.fallbacks = ws.xstate + 1;
    // the layer a decode loop calls next is, as a rule, the one after this one (and the first after the last)
    const size_t li = (size_t)(&L - h->layers.data()), nl = h->layers.size();
    if (h->warm_next && nl > 1 && li < nl) {
        const Layer &N = h->layers[(li + 1) % nl];
        if (N.router != nullptr) {
            lx.warm = N.router;
            lx.warm_bytes = (unsigned)((size_t)h->cfg.num_experts * (size_t)h->cfg.hidden_size * (N.router_type == T_F32 ? 4 : 2)) & ~15u;
        }
    }
    RouterExchange rx = router_exchange_of(h, L, ws, x, norm_gamma, xnorm_out);
    if (!decode_layer_supported(b, k, n, rx, lx)) return MUMMU_OK;
    RouteInline route;
    route.flavour = h->cfg.router_flavour;
    route.norm = norm;
    route.ids = ws.ids;
    route.weights = ws.weights;
    route.hits = L.hits;
    // A step of the chain of deferred sums: this launch adds up what the step before left, and leaves its own rows to the
    // next one.  It writes the set of buffers the pending step does not occupy.
    const float *xe = x + (size_t)n * (size_t)b.hidden;
    const bool chain = may_defer && h->deferred_combine && b.hidden % 256 == 0 && residual == nullptr && norm_gamma == nullptr;
    // (followed by a launch of its own for the sum the form is slower than two launches - 18.3 against 16.1 us per layer on
    // the OLMoE shape - so outside a chain it is taken only on request)
    if (!chain && h->layer_fusion < 2) return MUMMU_OK;
    PendingSum ps;
    if (h->pending.active) {
        const float *po = h->pending.out, *pe = po + (size_t)h->pending.n * (size_t)b.hidden;
        const bool x_is_pending = x < pe && po < xe;   // this step reads what the pending sum has yet to write
        if (!chain || h->pending.stream != s || x_is_pending) {
            const int rc = flush_pending(h);
            if (rc) return rc;
        } else {
            const DecodeBuffers pb = decode_buffers(h, h->pending.buf);
            ps.y = pb.y;
            ps.ids = pb.ids;
            ps.weights = pb.weights;
            ps.residual = h->pending.residual;
            ps.out = h->pending.out;
            ps.n = (int)h->pending.n;
        }
    }
    const int buf = chain ? h->decode_buf : 0;
    const DecodeBuffers db = decode_buffers(h, buf);
    lx.y = db.y;
    route.ids = db.ids;
    route.weights = db.weights;
    LAUNCH(h, K_DECODE_LAYER, s, launch_decode_layer(b, rx, lx, route, n, k, h->flags, s, ps));
    h->pending.active = false;
    h->routing_buf = buf;
    if (chain) {
        h->pending.active = true;
        h->pending.buf = buf;
        h->pending.k = k;
        h->pending.n = n;
        h->pending.residual = residual;
        h->pending.out = out;
        h->pending.stream = s;
        h->decode_buf = 1 - buf;
        // (the epoch of the exchange moves on with the next flush; until then the launches differ in their salt)
        if ((h->launch_salt & 0x3FFFFFFFu) == 0u) {
            const int rc = flush_pending(h);
            if (rc) return rc;
        }
    } else {
        LAUNCH(h, K_COMBINE, s, launch_combine(db.y, db.ids, db.weights, nullptr, n, k, b.hidden, residual, out, s, ws.xstate));
    }
    *done = true;
    return MUMMU_OK;
}

// The decode step in two launches where the device and the shapes allow it: router + routing + gate/up in one kernel
// (the workgroups exchange the logits inside it), then down + combine.  *done = false: not taken, nothing launched.
int decode_two_launches(mummu_moe *h, const Layer &L, const DecodeScratch &ws, const float *x, int n, int k, int norm,
                        const float *residual, float *out, hipStream_t s, const float *norm_gamma, float *xnorm_out, bool *done) {
    *done = false;
    if (!h->router_exchange || !h->xcd_round_robin || ws.xslots == nullptr || ws.xstate == nullptr) return MUMMU_OK;
    // measured on the OLMoE shape (Q4_K): one token 18.1 us against 18.4 in three launches, but 23.6 / 40.2 / 69.5 us
    // against 22.8 / 36.6 / 57.2 at 2 / 4 / 8 tokens - every workgroup repeats the router wait, and the fused kernel
    // keeps fewer waves per CU.  So one token only, unless a caller asks for it at every size (tests do).
    if (n > 1 && h->router_exchange < 2) return MUMMU_OK;
    const ExpertBanks b = banks_of(h, L);
    RouterExchange rx = router_exchange_of(h, L, ws, x, norm_gamma, xnorm_out);
    if (!gate_up_fused_supported(b, k, n, rx)) return MUMMU_OK;
    RouteInline route;
    route.flavour = h->cfg.router_flavour;
    route.norm = norm;
    route.ids = ws.ids;
    route.weights = ws.weights;
    route.hits = L.hits;
    LAUNCH(h, K_GATE_UP, s, launch_gate_up_fused(b, rx, route, n, k, ws.actq, h->flags, s));
    LAUNCH(h, K_DOWN_COMBINE, s, launch_down_combine(b, ws.actq, ws.ids, ws.weights, n, k, residual, out, s, ws.xstate));
    *done = true;
    return MUMMU_OK;
}

// norm_gamma != nullptr (only where decode_three_launches holds): x is the raw residual stream and the
// first launch applies the layer's RmsNorm itself.
int routed_impl(mummu_moe *h, int layer, const float *x, int64_t n, int k, int norm, const float *residual, float *out,
                hipStream_t s, const float *norm_gamma = nullptr, float *xnorm_out = nullptr, bool may_defer = false) {
    const Layer &L = h->layers[layer];
    const int E = h->cfg.num_experts, H = h->cfg.hidden_size;
    h->routing_buf = 0;
    if (!(may_defer && h->deferred_combine && n <= kExchangeTokens)) {  // (else the one-launch form decides: it may take the pending sum along)
        const int rc = flush_pending(h);
        if (rc) return rc;
    }
    // the fused router also quantizes x when the gate/up banks want it (whole 64-element slices)
    const bool batched = n >= batched_from(h, L);
    const bool want_xq = is_quant_type(L.gate_type) && H % 64 == 0 && !batched;
    const QAct xq = want_xq ? h->xq : QAct();
    if (norm_gamma && !decode_three_launches(h, L, n, k)) return fail(h, MUMMU_ERR_ARG, "fused RmsNorm outside the decode form");
    if (n > 8 && router_fused_supported(E)) {
        // many tokens: one workgroup per token tile does logits, routing and quantization
        // on the batched path the dispatch adds the per-expert row counts to the hit counters
        // ... and on the batched path with Q4_K banks on the f16 units it writes x as pairs of halfs beside the routing
        HAct xh;
        if (batched && !want_xq && router_converts_x((int)n, H, x, L.router)) xh = half_plan(h, banks_of(h, L), n, k).xh;
        LAUNCH(h, K_ROUTER, s,
               launch_router_fused(x, L.router, L.router_type, (int)n, H, E, k, h->cfg.router_flavour, norm, h->logits,
                                   h->ids, h->weights, batched ? nullptr : L.hits, h->flags, xq, s, xh));
        return run_experts(h, L, x, want_xq, n, k, residual, out, s, batched, xh.hi != nullptr);
    } else {
        if (want_xq) {
            const DecodeScratch ws{h->logits, h->ids, h->weights, h->xq, h->actq, h->xslots, h->xstate, h->aslots, h->y};
            bool done = false;
            int rc = decode_one_launch(h, L, ws, x, (int)n, k, norm, residual, out, s, norm_gamma, xnorm_out, may_defer, &done);
            if (rc || done) return rc;
            if ((rc = flush_pending(h))) return rc;
            rc = decode_two_launches(h, L, ws, x, (int)n, k, norm, residual, out, s, norm_gamma, xnorm_out, &done);
            if (rc || done) return rc;
        }
        {
            const int rc = flush_pending(h);
            if (rc) return rc;
        }
        // few tokens: the router rows are spread over as many CUs as there are experts
        LAUNCH(h, K_ROUTER_LOGITS, s,
               launch_router_logits(x, L.router, L.router_type, h->logits, (int)n, H, E, xq, s, norm_gamma, h->cfg.rms_norm_eps, xnorm_out));
        const ExpertBanks b = banks_of(h, L);
        if (want_xq && gate_up_routes_inline(b, k) && down_combine_supported(b, k)) {
            // ... and the gate/up kernel routes by itself: one launch less on the decode path
            const DecodeScratch ws{h->logits, h->ids, h->weights, h->xq, h->actq, nullptr, nullptr, nullptr, nullptr};
            return decode_tail(h, L, ws, (int)n, k, norm, residual, out, s);
        }
        if (!batched && float_decode_fused(b, k)) {
            // float banks: the same two fusions
            RouteInline route;
            route.logits = h->logits;
            route.flavour = h->cfg.router_flavour;
            route.norm = norm;
            route.ids = h->ids;
            route.weights = h->weights;
            route.hits = L.hits;
            LAUNCH(h, K_GATE_UP, s, launch_gate_up_f_routed(b, x, route, (int)n, k, h->act, h->flags, s));
            LAUNCH(h, K_DOWN_COMBINE, s, launch_down_combine_f(b, h->act, h->ids, h->weights, (int)n, k, residual, out, s));
            return MUMMU_OK;
        }
        LAUNCH(h, K_ROUTE_TOPK, s,
               launch_route_topk(h->logits, (int)n, E, k, h->cfg.router_flavour, norm, h->ids, h->weights, L.hits, h->flags, s));
    }
    return run_experts(h, L, x, want_xq, n, k, residual, out, s);
}

// The block: the routed experts, plus (when the layer has one) the shared expert every token
// takes, scaled by its sigmoid gate (models/qwen4exp/model.rs:786-804):
//     out = [residual +] (routed + shared_ffn(x) * sigmoid(<gate_vec, x>))
// with the product and the two sums rounded separately, in that grouping.
int forward_impl(mummu_moe *h, int layer, const float *x, int64_t n, int k, int norm, const float *residual, float *out,
                 hipStream_t s, const float *norm_gamma = nullptr, bool may_defer = false) {
    const Layer &L = h->layers[layer];
    if (!L.sh_loaded) return routed_impl(h, layer, x, n, k, norm, residual, out, s, norm_gamma, nullptr, may_defer);
    // with the RmsNorm inside the router launch the shared expert reads the normalised rows that launch leaves in h2
    const float *x_raw = x;
    if (norm_gamma) x = h->h2;
    if (n > h->sh_ws_tokens) return fail(h, MUMMU_ERR_TOKENS, "shared-expert workspace is smaller than the call");
    const int H = h->cfg.hidden_size;
    ExpertBanks b;
    b.gate = L.sh_gate;
    b.up = L.sh_up;
    b.down = L.sh_down;
    b.gate_type = L.sh_gate_type;
    b.up_type = L.sh_up_type;
    b.down_type = L.sh_down_type;
    b.hidden = H;
    b.inter = L.sh_inter;
    b.n_experts = 1;
    const int sh_from = !grouped_gemm_supported(b) ? 0x7fffffff
                        : (b.gate_type == T_F32 ? h->gemm_min_f32 : (grouped_gemm_quantized(b) ? h->gemm_min_quant : h->gemm_min_f16));
    // (one expert makes few workgroups: tiles x 128-row slabs.  Measured at H 2048, shared inter 2048, Q4_K: the
    // per-token kernels cost 68 us at 64 tokens and 396 us at 512, the GEMM pair about 145 us at either)
    int rc = norm_gamma ? routed_impl(h, layer, x_raw, n, k, norm, nullptr, out, s, norm_gamma, h->h2)
                        : routed_impl(h, layer, x, n, k, norm, nullptr, out, s);
    if (rc) return rc;
    if (n >= sh_from && n >= 192) {
        // many tokens: the shared expert is one more grouped GEMM pair, every row in order on expert 0
        const int tile_rows = grouped_gemm_tile_rows(b, (int)n, 1);
        const QAct64 xq64{h->xq.hi, h->xq.lo, h->xq.scale, (float *)h->xq.sum};
        const QAct64 actq64{h->sh_actq.hi, h->sh_actq.lo, h->sh_actq.scale, (float *)h->sh_actq.sum};
        LAUNCH(h, K_SHARED, s, launch_identity_tiles((int)n, tile_rows, h->sh_sorted, h->sh_tiles, h->sh_ntiles, s));
        // (the routed path may have left the 16-bit activations in the decode layout, or not made them)
        // (Q4_K on the f16 units as in the routed path; the routed products are done with their output buffer)
        const bool small32 = (size_t)n * (size_t)(b.hidden > b.inter ? b.hidden : b.inter) * 2 < (1ull << 32);
        const bool hf = h->gemm_q4k_f16 && small32 && grouped_gemm_q4k_f16(b), hf_down = hf && grouped_gemm_q4k_f16_down(b);
        const bool half_banks = b.gate_type == T_F16 || b.gate_type == T_BF16;
        const HAct xh = hf ? HAct{(_Float16 *)h->sh_y, (_Float16 *)h->sh_y + (size_t)n * H, h->xq.scale, (float *)h->xq.sum}
                           : (half_banks ? HAct{(_Float16 *)h->sh_y, nullptr, nullptr, nullptr} : HAct());
        const HAct acth = hf_down ? HAct{(_Float16 *)h->sh_act16, (_Float16 *)h->sh_act, h->sh_actq.scale, (float *)h->sh_actq.sum} : HAct();
        if (hf) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows_h(x, (int)n, H, xh, s));
        else if (half_banks) LAUNCH(h, K_QUANTIZE, s, launch_convert_rows_f16(x, (int)n, H, xh.hi, s));
        else if (grouped_gemm_quantized(b)) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows64(x, (int)n, H, xq64, s));
        LAUNCH(h, K_SHARED, s,
               launch_gemm_gate_up(b, x, xq64, xh, h->sh_sorted, 1, h->sh_tiles, h->sh_ntiles, h->sh_max_tiles, tile_rows, h->sh_act16,
                                   h->sh_act, actq64, acth, s));
        LAUNCH(h, K_SHARED, s,
               launch_gemm_down(b, h->sh_act16, h->sh_act, actq64, acth, (int)n, h->sh_tiles, h->sh_ntiles, h->sh_max_tiles, tile_rows,
                                h->sh_y, s));
    } else {
        // the routed decode kernels leave x in the 16-bit decode layout when their own banks are quantized;
        // otherwise (float routed banks, or the batched path's layout) it is made here
        const bool have_xq = is_quant_type(L.gate_type) && H % 64 == 0 && n < batched_from(h, L);
        if (is_quant_type(b.gate_type) && !have_xq) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows(x, (int)n, H, h->xq, s));
        LAUNCH(h, K_SHARED, s, launch_gate_up(b, x, h->xq, nullptr, (int)n, 1, 0, h->sh_act, h->sh_actq, h->flags, s));
        LAUNCH(h, K_SHARED, s, launch_down(b, h->sh_act, h->sh_actq, nullptr, (int)n, 1, 0, h->sh_y, s));
    }
    LAUNCH(h, K_SHARED, s, launch_shared_add(out, h->sh_y, x, L.sh_gatevec, L.sh_gatevec_type, residual, (int)n, H, s));
    return MUMMU_OK;
}

int check_device_call(mummu_moe *h, int64_t n, int k, const void *a, const void *b) {
    if (!a || !b) return fail(h, MUMMU_ERR_ARG, "null device pointer");
    if (((uintptr_t)a & 15) || ((uintptr_t)b & 15)) return fail(h, MUMMU_ERR_ARG, "device buffers must be 16-byte aligned");
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n > h->ws_tokens || n * k > h->ws_assign)
        return fail(h, MUMMU_ERR_TOKENS, std::to_string(n) + " tokens x top_k " + std::to_string(k) +
                                             " exceeds the workspace (max_tokens " + std::to_string(h->ws_tokens) + ", pairs " +
                                             std::to_string(h->ws_assign) + ")");
    return MUMMU_OK;
}

// Do workgroups whose linear ids agree modulo 8 run on one XCD?  (The router exchange splits its work on that
// assumption; it stays correct without it, only slow, so it is switched off then.)  Probed with the launch shape of the
// decode kernels.
__global__ __launch_bounds__(256) void xcd_probe_kernel(int *out) {
    if (threadIdx.x == 0)
        out[blockIdx.y * gridDim.x + blockIdx.x] = (int)(__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u);  // HW_REG_XCC_ID[3:0]
}

int probe_xcd_round_robin(mummu_moe *h) {
    constexpr int kProbe = 512;
    int *d = nullptr;
    HIPCHK(h, hipMalloc((void **)&d, sizeof(int) * kProbe));
    std::vector<int> got(kProbe);
    bool rr = true;
    hipError_t e = hipSuccess;
    for (int rep = 0; rep < 2 && e == hipSuccess; rep++) {
        launch_kernel(xcd_probe_kernel, dim3(8, kProbe / 8), dim3(256), 0, h->stream, d);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipMemcpyAsync(got.data(), d, sizeof(int) * kProbe, hipMemcpyDeviceToHost, h->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
        for (int i = 0; i < kProbe && e == hipSuccess; i++) rr = rr && got[i] == got[i & 7];
    }
    (void)hipFree(d);
    if (e != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("XCD probe: ") + hipGetErrorString(e));
    if (getenv("MUMMU_DEBUG")) {
        fprintf(stderr, "[mummu] XCD of workgroups 0..15:");
        for (int i = 0; i < 16; i++) fprintf(stderr, " %d", got[i]);
        fprintf(stderr, "  -> same XCD for equal id mod 8: %s\n", rr ? "yes" : "no");
    }
    h->xcd_round_robin = rr;
    return MUMMU_OK;
}

int stack_impl(mummu_moe *h, const float *x, int64_t n, int k, int norm, float *out, hipStream_t s, int32_t *ids_host) {
    const int nl = (int)h->layers.size(), H = h->cfg.hidden_size;
    {
        const int rc = flush_pending(h);
        if (rc) return rc;
    }
    for (int l = 0; l < nl; l++) {
        int rc = check_layer(h, l);
        if (rc) return rc;
        if (!h->layers[l].gamma) return fail(h, MUMMU_ERR_NOT_LOADED, "layer " + std::to_string(l) + " has no RmsNorm weight");
    }
    for (int l = 0; l < nl; l++) {
        const float *src = l == 0 ? x : h->resid[(l - 1) & 1];
        float *dst = l == nl - 1 ? out : h->resid[l & 1];
        const Layer &L = h->layers[l];
        int rc;
        if (decode_three_launches(h, L, n, k) && router_logits_can_norm(src, L.router, L.gamma, (int)n, H)) {
            // decode: the router launch normalises the row it already holds; no launch of its own
            rc = forward_impl(h, l, src, n, k, norm, src, dst, s, L.gamma);
        } else {
            LAUNCH(h, K_RMSNORM, s, launch_rmsnorm(src, L.gamma, h->cfg.rms_norm_eps, (int)n, H, h->h2, s));
            rc = forward_impl(h, l, h->h2, n, k, norm, src, dst, s);
        }
        if (rc) return rc;
        if (ids_host) {
            HIPCHK(h, hipStreamSynchronize(s));
            HIPCHK(h, hipMemcpy(ids_host + (size_t)l * n * k, decode_buffers(h, h->routing_buf).ids, sizeof(int32_t) * (size_t)(n * k),
                                hipMemcpyDeviceToHost));
        }
    }
    return MUMMU_OK;
}

}  // namespace

namespace mummu {

// 16-bit rows <-> f32 rows for the entry point that takes the caller's ambient dtype.  Widening is exact;
// narrowing rounds to nearest even (NaN stays NaN).
template <int T>
__global__ __launch_bounds__(256) void widen_rows_kernel(const uint16_t *__restrict__ src, size_t n, float *__restrict__ dst) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = T == T_F16 ? half_bits_to_float(src[i]) : bf16_bits_to_float(src[i]);
}

template <int T>
__global__ __launch_bounds__(256) void narrow_rows_kernel(const float *__restrict__ src, size_t n, uint16_t *__restrict__ dst) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = src[i];
    if (T == T_F16) {
        dst[i] = __builtin_bit_cast(uint16_t, (_Float16)v);  // round to nearest even
    } else {
        const uint32_t b = __float_as_uint(v);
        dst[i] = v != v ? (uint16_t)((b >> 16) | 0x0040u) : (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
    }
}

}  // namespace mummu

extern "C" {

int mummu_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

const char *mummu_moe_last_error(const mummu_moe *h) { return h ? h->err.c_str() : g_error.c_str(); }

int mummu_moe_create(const mummu_moe_config *cfg, mummu_moe **out) {
    if (!cfg || !out) return fail(nullptr, MUMMU_ERR_ARG, "null config or output pointer");
    *out = nullptr;
    // nn/moe.rs:62-76
    if (cfg->num_experts < 2)
        return fail(nullptr, MUMMU_ERR_CONFIG,
                    "MoE: num_experts must be >= 2 (got " + std::to_string(cfg->num_experts) + "); use SwiGluMlp for a dense FFN");
    if (cfg->num_experts_per_tok < 1 || cfg->num_experts_per_tok > cfg->num_experts)
        return fail(nullptr, MUMMU_ERR_CONFIG, "MoE: num_experts_per_tok (" + std::to_string(cfg->num_experts_per_tok) +
                                                   ") must be in 1..=num_experts (" + std::to_string(cfg->num_experts) + ")");
    if (cfg->hidden_size < 1 || cfg->expert_intermediate_size < 1)
        return fail(nullptr, MUMMU_ERR_CONFIG, "MoE: hidden_size and expert_intermediate_size must be >= 1");
    if (cfg->num_experts > 512) return fail(nullptr, MUMMU_ERR_CONFIG, "MoE: this build routes over at most 512 experts");
    if (cfg->num_layers < 1 || cfg->max_tokens < 1) return fail(nullptr, MUMMU_ERR_CONFIG, "MoE: num_layers and max_tokens must be >= 1");
    if (cfg->router_flavour != MUMMU_ROUTER_SPARSE_MOE && cfg->router_flavour != MUMMU_ROUTER_QWEN4EXP)
        return fail(nullptr, MUMMU_ERR_CONFIG, "MoE: unknown router_flavour");
    if (mummu_device_count() < 1) return fail(nullptr, MUMMU_ERR_DEVICE, "no HIP device visible to this process");

    mummu_moe *h = new mummu_moe();
    h->cfg = *cfg;
    // MUMMU_GEMM_Q4K_F16=0: Q4_K banks of the batched path stay on the int8 units (the form every other block-quantized
    // type takes) instead of the f16 units
    if (const char *e = getenv("MUMMU_GEMM_Q4K_F16")) h->gemm_q4k_f16 = atoi(e) != 0;
    // MUMMU_GEMM_Q8_F16=1: Q8_0 banks of the batched path take the f16 kernel (every weight exact as two halfs, x and the
    // activations between the products rounded to halfs as for F16 banks: 1.2 to 1.5 times faster, errors of 1.5e-3
    // by the reference's measure where the int8 form has 2e-4 - which is why it is not the default)
    if (const char *e = getenv("MUMMU_GEMM_Q8_F16")) h->gemm_q8_f16 = atoi(e) != 0;
    // MUMMU_GEMM_TILE_ROWS=16 | 32 | 64: rows per tile of the f16-unit Q4_K kernels (default: by expected cost)
    if (const char *e = getenv("MUMMU_GEMM_TILE_ROWS")) {
        const int v = atoi(e);
        if (v == 16 || v == 32 || v == 64) h->gemm_tile_rows = v;
    }
    // MUMMU_GEMM_MIN_TOKENS: smallest batch that takes dispatch + grouped GEMM instead of the decode kernels
    if (const char *e = getenv("MUMMU_GEMM_MIN_TOKENS")) {
        const int v = atoi(e);
        if (v >= 1) h->gemm_min_f16 = h->gemm_min_quant = h->gemm_min_f32 = h->gemm_min_q4k = v;
    }
    h->layers.resize((size_t)cfg->num_layers);
    auto bail = [&](int rc) {
        g_error = h->err;
        mummu_moe_destroy(h);
        return rc;
    };
    if (hipSetDevice(0) != hipSuccess) return bail(fail(h, MUMMU_ERR_DEVICE, "hipSetDevice(0) failed"));
    if (hipStreamCreate(&h->stream) != hipSuccess) return bail(fail(h, MUMMU_ERR_DEVICE, "hipStreamCreate failed"));
    if (hipHostMalloc((void **)&h->pin, 2 * kPinIO + 64, hipHostMallocDefault) != hipSuccess) {
        h->pin = nullptr;  // not fatal: the calls then copy straight from the caller's memory
        (void)hipGetLastError();
    }
    if (hipEventCreate(&h->t0) != hipSuccess || hipEventCreate(&h->t1) != hipSuccess)
        return bail(fail(h, MUMMU_ERR_DEVICE, "hipEventCreate failed"));
    if (hipMalloc(&h->flags, sizeof(int32_t) * kFlagWords) != hipSuccess) return bail(fail(h, MUMMU_ERR_DEVICE, "hipMalloc(flags) failed"));
    int rc = reset_flags(h);
    if (rc) return bail(rc);
    {
        // the router exchange: table and state, and whether workgroups land on the XCDs the way it assumes
        const size_t xb = router_exchange_bytes(cfg->num_experts);
        if (hipMalloc(&h->xslots, xb) != hipSuccess || hipMalloc((void **)&h->xstate, 256) != hipSuccess)
            return bail(fail(h, MUMMU_ERR_DEVICE, "hipMalloc(router exchange) failed"));
        if (hipMemset(h->xslots, 0, xb) != hipSuccess || hipMemset(h->xstate, 0, 256) != hipSuccess)
            return bail(fail(h, MUMMU_ERR_DEVICE, "hipMemset(router exchange) failed"));
        if (hipMalloc(&h->aslots, layer_exchange_bytes()) != hipSuccess || hipMemset(h->aslots, 0, layer_exchange_bytes()) != hipSuccess)
            return bail(fail(h, MUMMU_ERR_DEVICE, "hipMalloc(hidden-row exchange) failed"));
        if ((rc = probe_xcd_round_robin(h))) return bail(rc);
        if (const char *e = getenv("MUMMU_ROUTER_EXCHANGE")) h->router_exchange = atoi(e) < 0 ? 0 : (atoi(e) > 2 ? 2 : atoi(e));
        if (const char *e = getenv("MUMMU_LAYER_FUSION")) h->layer_fusion = atoi(e) < 0 ? 0 : (atoi(e) > 2 ? 2 : atoi(e));
        if (const char *e = getenv("MUMMU_DEFERRED_COMBINE")) h->deferred_combine = atoi(e) != 0;
        if (const char *e = getenv("MUMMU_TILE_ORDER")) h->tile_order = atoi(e) < 0 ? -1 : (atoi(e) != 0);
        if (const char *e = getenv("MUMMU_EARLY_IDS")) h->early_ids = atoi(e) != 0;
        if (const char *e = getenv("MUMMU_WARM_NEXT")) h->warm_next = atoi(e) != 0;
    }
    {
        // resolve the static scratch's address on this device now, outside any stream capture
        unsigned char *unused = nullptr;
        if ((rc = static_scratch(h, &unused))) return bail(rc);
    }
    rc = ensure_ws(h, cfg->max_tokens, (int64_t)cfg->max_tokens * cfg->num_experts_per_tok, cfg->num_experts);
    if (rc) return bail(rc);
    *out = h;
    return MUMMU_OK;
}

void mummu_moe_destroy(mummu_moe *h) {
    if (!h) return;
    (void)flush_pending(h);
    (void)hipDeviceSynchronize();
    for (Layer &L : h->layers) {
        void *ptrs[] = {L.router, L.gate, L.up, L.down, L.gamma, L.hits, L.sh_gate, L.sh_up, L.sh_down, L.sh_gatevec};
        for (void *p : ptrs)
            if (p) (void)hipFree(p);
    }
    free_ws(h);
    if (h->xslots) (void)hipFree(h->xslots);
    if (h->xstate) (void)hipFree(h->xstate);
    if (h->aslots) (void)hipFree(h->aslots);
    if (h->flags) (void)hipFree(h->flags);
    for (auto &t : h->timed) {
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    for (auto e : h->event_pool) (void)hipEventDestroy(e);
    if (h->t0) (void)hipEventDestroy(h->t0);
    if (h->t1) (void)hipEventDestroy(h->t1);
    if (h->pin) (void)hipHostFree(h->pin);
    if (h->stream) (void)hipStreamDestroy(h->stream);
    delete h;
}

int mummu_moe_load_layer(mummu_moe *h, int layer, const void *router, int router_type, const void *gate, int gate_type,
                         const void *up, int up_type, const void *down, int down_type, const float *rms_gamma) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    if (layer < 0 || layer >= (int)h->layers.size())
        return fail(h, MUMMU_ERR_RANGE, "layer " + std::to_string(layer) + " out of range (" + std::to_string(h->layers.size()) + ")");
    if (!router || !gate || !up || !down) return fail(h, MUMMU_ERR_ARG, "null weight pointer");
    if (!router_type_ok(router_type)) return fail(h, MUMMU_ERR_TYPE, "router must be F32, F16 or BF16 (got ggml type " + std::to_string(router_type) + ")");
    for (int t : {gate_type, up_type, down_type})
        if (!bank_type_ok(t)) return fail(h, MUMMU_ERR_TYPE, "no expert kernel for ggml type " + std::to_string(t));
    if (gate_type != up_type) return fail(h, MUMMU_ERR_TYPE, "gate and up banks must share one type");
    const int H = h->cfg.hidden_size, I = h->cfg.expert_intermediate_size, E = h->cfg.num_experts;
    // experts.rs:150-154: a row that is not whole blocks cannot be sliced out of the bank
    if (H % block_elems(gate_type))
        return fail(h, MUMMU_ERR_BLOCKS, "row width " + std::to_string(H) + " is not whole blocks of " + std::to_string(block_elems(gate_type)));
    if (I % block_elems(down_type))
        return fail(h, MUMMU_ERR_BLOCKS, "row width " + std::to_string(I) + " is not whole blocks of " + std::to_string(block_elems(down_type)));
    if (is_quant_type(gate_type) && H / 32 > 256)
        return fail(h, MUMMU_ERR_CONFIG, "quantized rows wider than 8192 are not supported");
    if (is_quant_type(down_type) && I / 32 > 256)
        return fail(h, MUMMU_ERR_CONFIG, "quantized rows wider than 8192 are not supported");

    Layer &L = h->layers[layer];
    HIPCHK(h, hipDeviceSynchronize());
    if (L.loaded) h->generation++;
    void *old[] = {L.router, L.gate, L.up, L.down, L.gamma, L.hits, L.sh_gate, L.sh_up, L.sh_down, L.sh_gatevec};
    for (void *p : old)
        if (p) (void)hipFree(p);
    L = Layer();
    const size_t rb = (size_t)E * (size_t)H * (size_t)block_bytes(router_type);
    const size_t gb = (size_t)E * (size_t)I * row_bytes_of(gate_type, H);
    const size_t ub = (size_t)E * (size_t)I * row_bytes_of(up_type, H);
    const size_t db = (size_t)E * (size_t)H * row_bytes_of(down_type, I);
    HIPCHK(h, hipMalloc(&L.router, rb));
    HIPCHK(h, hipMalloc(&L.gate, gb));
    HIPCHK(h, hipMalloc(&L.up, ub));
    HIPCHK(h, hipMalloc(&L.down, db));
    HIPCHK(h, hipMalloc(&L.hits, sizeof(unsigned long long) * (size_t)E));
    HIPCHK(h, hipMemcpy(L.router, router, rb, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemcpy(L.gate, gate, gb, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemcpy(L.up, up, ub, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemcpy(L.down, down, db, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemset(L.hits, 0, sizeof(unsigned long long) * (size_t)E));
    if (rms_gamma) {
        HIPCHK(h, hipMalloc(&L.gamma, sizeof(float) * (size_t)H));
        HIPCHK(h, hipMemcpy(L.gamma, rms_gamma, sizeof(float) * (size_t)H, hipMemcpyHostToDevice));
    }
    L.router_type = router_type;
    L.gate_type = gate_type;
    L.up_type = up_type;
    L.down_type = down_type;
    if (gate_type == T_Q8_0 && up_type == T_Q8_0 && down_type == T_Q8_0) {
        // the f16 kernel multiplies d * code as halfs: only banks whose largest |d| * 128 is a finite half (|d| < 512: a code may be -128)
        uint32_t *max_bits = nullptr, got = 0;
        HIPCHK(h, hipMalloc((void **)&max_bits, sizeof(uint32_t)));
        hipError_t e = hipMemsetAsync(max_bits, 0, sizeof(uint32_t), h->stream);
        if (e == hipSuccess) e = launch_q8_scale_max(L.gate, gb / 34, max_bits, h->stream);
        if (e == hipSuccess) e = launch_q8_scale_max(L.up, ub / 34, max_bits, h->stream);
        if (e == hipSuccess) e = launch_q8_scale_max(L.down, db / 34, max_bits, h->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
        if (e == hipSuccess) e = hipMemcpy(&got, max_bits, sizeof(uint32_t), hipMemcpyDeviceToHost);
        (void)hipFree(max_bits);
        HIPCHK(h, e);
        L.q8_half_ok = got < 0x6000u;   // half bits of 512.0: 512 * -128 = -65536 rounds to -inf
    }
    L.bytes = rb + gb + ub + db + (rms_gamma ? sizeof(float) * (size_t)H : 0);
    L.loaded = true;
    return MUMMU_OK;
}

int mummu_moe_load_shared_expert(mummu_moe *h, int layer, int inter, const void *gate, int gate_type, const void *up, int up_type,
                                 const void *down, int down_type, const void *gate_vec, int gate_vec_type) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);  // the routed part of the layer comes first
    if (rc) return rc;
    if (!gate || !up || !down) return fail(h, MUMMU_ERR_ARG, "null weight pointer");
    for (int t : {gate_type, up_type, down_type})
        if (!bank_type_ok(t)) return fail(h, MUMMU_ERR_TYPE, "no expert kernel for ggml type " + std::to_string(t));
    if (gate_type != up_type) return fail(h, MUMMU_ERR_TYPE, "gate and up banks must share one type");
    if (gate_vec && !router_type_ok(gate_vec_type))
        return fail(h, MUMMU_ERR_TYPE, "the shared expert's gate vector must be F32, F16 or BF16 (got ggml type " + std::to_string(gate_vec_type) + ")");
    const int H = h->cfg.hidden_size;
    if (inter < 1) return fail(h, MUMMU_ERR_CONFIG, "shared expert width must be >= 1");
    if (H % block_elems(gate_type))
        return fail(h, MUMMU_ERR_BLOCKS, "row width " + std::to_string(H) + " is not whole blocks of " + std::to_string(block_elems(gate_type)));
    if (inter % block_elems(down_type))
        return fail(h, MUMMU_ERR_BLOCKS, "row width " + std::to_string(inter) + " is not whole blocks of " + std::to_string(block_elems(down_type)));
    if ((is_quant_type(gate_type) && H / 32 > 256) || (is_quant_type(down_type) && inter / 32 > 256))
        return fail(h, MUMMU_ERR_CONFIG, "quantized rows wider than 8192 are not supported");
    if (is_quant_type(down_type) && inter % 16) return fail(h, MUMMU_ERR_BLOCKS, "shared expert width must be a multiple of 16 for a quantized down matrix");
    Layer &L = h->layers[layer];
    HIPCHK(h, hipDeviceSynchronize());
    h->generation++;  // a graph captured before this call does not run the shared expert (or points at the old one)
    void *old[] = {L.sh_gate, L.sh_up, L.sh_down, L.sh_gatevec};
    for (void *p : old)
        if (p) (void)hipFree(p);
    L.sh_gate = L.sh_up = L.sh_down = nullptr;
    L.sh_gatevec = nullptr;
    L.sh_loaded = false;
    L.sh_bytes = 0;
    const size_t gb = (size_t)inter * row_bytes_of(gate_type, H), db = (size_t)H * row_bytes_of(down_type, inter);
    const size_t vb = gate_vec ? (size_t)H * (size_t)block_bytes(gate_vec_type) : 0;
    HIPCHK(h, hipMalloc(&L.sh_gate, gb));
    HIPCHK(h, hipMalloc(&L.sh_up, gb));
    HIPCHK(h, hipMalloc(&L.sh_down, db));
    HIPCHK(h, hipMemcpy(L.sh_gate, gate, gb, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemcpy(L.sh_up, up, gb, hipMemcpyHostToDevice));
    HIPCHK(h, hipMemcpy(L.sh_down, down, db, hipMemcpyHostToDevice));
    if (gate_vec) {
        HIPCHK(h, hipMalloc(&L.sh_gatevec, vb));
        HIPCHK(h, hipMemcpy(L.sh_gatevec, gate_vec, vb, hipMemcpyHostToDevice));
    }
    L.sh_gate_type = gate_type;
    L.sh_up_type = up_type;
    L.sh_down_type = down_type;
    L.sh_gatevec_type = gate_vec_type;
    L.sh_inter = inter;
    L.sh_bytes = 2 * gb + db + vb;
    L.sh_loaded = true;
    if (inter > h->sh_inter_max) {
        h->sh_inter_max = inter;
        h->sh_ws_tokens = 0;  // regrow for the wider expert
    }
    return ensure_shared_ws(h);
}

int mummu_moe_batched_from(const mummu_moe *h, int layer) {
    if (!h || layer < 0 || layer >= (int)h->layers.size() || !h->layers[layer].loaded) return 0x7fffffff;
    return batched_from(h, h->layers[layer]);
}

int mummu_moe_get_config(const mummu_moe *h, mummu_moe_config *out) {
    if (!h || !out) return fail(nullptr, MUMMU_ERR_ARG, "null argument");
    *out = h->cfg;
    return MUMMU_OK;
}

uint64_t mummu_moe_resident_bytes(const mummu_moe *h) {
    if (!h) return 0;
    uint64_t total = 0;
    for (const Layer &L : h->layers) total += L.bytes + L.sh_bytes;
    return total;
}

int mummu_moe_forward(mummu_moe *h, int layer, const float *x, int64_t n, int top_k, int norm, float *out) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!x || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    const size_t bytes = sizeof(float) * (size_t)n * (size_t)h->cfg.hidden_size;
    if ((rc = upload_rows(h, h->xin, x, bytes, h->stream))) return rc;
    if ((rc = forward_impl(h, layer, h->xin, n, top_k, norm, nullptr, h->xout, h->stream))) return rc;
    return download_rows(h, out, h->xout, bytes, h->stream, true);
}

int mummu_moe_forward_typed(mummu_moe *h, int layer, const void *x, int x_type, int64_t n, int top_k, int norm, void *out) {
    if (x_type == MUMMU_F32) return mummu_moe_forward(h, layer, (const float *)x, n, top_k, norm, (float *)out);
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    if (x_type != MUMMU_F16 && x_type != MUMMU_BF16)
        return fail(h, MUMMU_ERR_TYPE, "forward: activations are F32, F16 or BF16 (got type " + std::to_string(x_type) + ")");
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!x || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    hipStream_t s = h->stream;
    const size_t count = (size_t)n * (size_t)h->cfg.hidden_size, bytes16 = count * 2;
    const dim3 grid((unsigned)((count + 255) / 256)), block(256);
    // the 16-bit rows land in the output buffer (not yet needed), are widened into the input buffer, and after the
    // block has run the f32 result is narrowed into the input buffer (no longer needed) and read back from there
    if ((rc = upload_rows(h, h->xout, (const float *)x, bytes16, s))) return rc;
    if (x_type == MUMMU_F16) launch_kernel(widen_rows_kernel<T_F16>, grid, block, 0, s, (const uint16_t *)h->xout, count, h->xin);
    else launch_kernel(widen_rows_kernel<T_BF16>, grid, block, 0, s, (const uint16_t *)h->xout, count, h->xin);
    HIPCHK(h, hipGetLastError());
    if ((rc = forward_impl(h, layer, h->xin, n, top_k, norm, nullptr, h->xout, s))) return rc;
    if (x_type == MUMMU_F16) launch_kernel(narrow_rows_kernel<T_F16>, grid, block, 0, s, (const float *)h->xout, count, (uint16_t *)h->xin);
    else launch_kernel(narrow_rows_kernel<T_BF16>, grid, block, 0, s, (const float *)h->xout, count, (uint16_t *)h->xin);
    HIPCHK(h, hipGetLastError());
    return download_rows(h, (float *)out, h->xin, bytes16, s, true);
}

int mummu_moe_route(mummu_moe *h, int layer, const float *x, int64_t n, int top_k, int norm, int32_t *ids, float *weights,
                    float *logits) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!x || !ids || !weights) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    const Layer &L = h->layers[layer];
    const int E = h->cfg.num_experts, H = h->cfg.hidden_size;
    hipStream_t s = h->stream;
    HIPCHK(h, hipMemcpyAsync(h->xin, x, sizeof(float) * (size_t)n * H, hipMemcpyHostToDevice, s));
    LAUNCH(h, K_ROUTER_LOGITS, s, launch_router_logits(h->xin, L.router, L.router_type, h->logits, (int)n, H, E, QAct(), s));
    LAUNCH(h, K_ROUTE_TOPK, s,
           launch_route_topk(h->logits, (int)n, E, top_k, h->cfg.router_flavour, norm, h->ids, h->weights, nullptr, h->flags, s));
    return download_routing(h, ids, weights, (size_t)(n * top_k), logits, (size_t)n * (size_t)E, s);
}

int mummu_route_logits(mummu_moe *h, const float *logits, int64_t n, int n_experts, int top_k, int flavour, int norm,
                       int32_t *ids, float *weights) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    // experts.rs:542-544
    if (n_experts <= 0 || top_k <= 0 || top_k > n_experts)
        return fail(h, MUMMU_ERR_TOPK, "top-" + std::to_string(top_k) + " of " + std::to_string(n_experts) + " experts is not a routing");
    if (n_experts > 512) return fail(h, MUMMU_ERR_CONFIG, "this build routes over at most 512 experts");
    if (flavour != MUMMU_ROUTER_SPARSE_MOE && flavour != MUMMU_ROUTER_QWEN4EXP) return fail(h, MUMMU_ERR_CONFIG, "unknown router flavour");
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!logits || !ids || !weights) return fail(h, MUMMU_ERR_ARG, "null buffer");
    int rc = ensure_ws(h, n, n * top_k, n_experts);
    if (rc) return rc;
    hipStream_t s = h->stream;
    HIPCHK(h, hipMemcpyAsync(h->logits, logits, sizeof(float) * (size_t)n * n_experts, hipMemcpyHostToDevice, s));
    LAUNCH(h, K_ROUTE_TOPK, s, launch_route_topk(h->logits, (int)n, n_experts, top_k, flavour, norm, h->ids, h->weights, nullptr, h->flags, s));
    HIPCHK(h, hipStreamSynchronize(s));
    int32_t f[4];
    HIPCHK(h, hipMemcpy(f, h->flags, sizeof(f), hipMemcpyDeviceToHost));
    if (f[FLAG_NONFINITE]) {
        if ((rc = reset_flags(h))) return rc;
        char buf[160];
        snprintf(buf, sizeof(buf), "router logit for token %d expert %d is not finite", f[FLAG_NONFINITE_INDEX] / n_experts,
                 f[FLAG_NONFINITE_INDEX] % n_experts);
        return fail(h, MUMMU_ERR_NONFINITE, buf);
    }
    HIPCHK(h, hipMemcpy(ids, h->ids, sizeof(int32_t) * (size_t)(n * top_k), hipMemcpyDeviceToHost));
    HIPCHK(h, hipMemcpy(weights, h->weights, sizeof(float) * (size_t)(n * top_k), hipMemcpyDeviceToHost));
    return MUMMU_OK;
}

int mummu_moe_apply_routing(mummu_moe *h, int layer, const int32_t *ids, const float *weights, const float *xs, int64_t n,
                            int top_k, float *out) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!ids || !weights || !xs || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    // experts.rs:1111-1117
    for (int64_t i = 0; i < n * top_k; i++)
        if (ids[i] < 0 || ids[i] >= h->cfg.num_experts)
            return fail(h, MUMMU_ERR_RANGE, "routed expert " + std::to_string(ids[i]) + " out of range (" + std::to_string(h->cfg.num_experts) + ")");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    hipStream_t s = h->stream;
    const size_t bytes = sizeof(float) * (size_t)n * (size_t)h->cfg.hidden_size;
    HIPCHK(h, hipMemcpyAsync(h->xin, xs, bytes, hipMemcpyHostToDevice, s));
    HIPCHK(h, hipMemcpyAsync(h->ids, ids, sizeof(int32_t) * (size_t)(n * top_k), hipMemcpyHostToDevice, s));
    HIPCHK(h, hipMemcpyAsync(h->weights, weights, sizeof(float) * (size_t)(n * top_k), hipMemcpyHostToDevice, s));
    Layer &L = h->layers[layer];
    // hit counters, nn/moe.rs:1562-1564 (the routing came from the host, so count here)
    {
        std::vector<unsigned long long> add((size_t)h->cfg.num_experts, 0), cur((size_t)h->cfg.num_experts);
        for (int64_t i = 0; i < n * top_k; i++) add[(size_t)ids[i]]++;
        HIPCHK(h, hipStreamSynchronize(s));
        HIPCHK(h, hipMemcpy(cur.data(), L.hits, sizeof(unsigned long long) * cur.size(), hipMemcpyDeviceToHost));
        for (size_t e = 0; e < cur.size(); e++) cur[e] += add[e];
        HIPCHK(h, hipMemcpy(L.hits, cur.data(), sizeof(unsigned long long) * cur.size(), hipMemcpyHostToDevice));
    }
    if ((rc = run_experts(h, L, h->xin, false, n, top_k, nullptr, h->xout, s))) return rc;
    return download_rows(h, out, h->xout, bytes, s, true);
}

int mummu_moe_routed(mummu_moe *h, int layer, const float *router_logits, const float *xs, int64_t n, int top_k, float *out) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (n <= 0) return n < 0 ? fail(h, MUMMU_ERR_SHAPE, "negative token count") : MUMMU_OK;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (!router_logits || !xs || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    // route on the device from the caller's logits (experts.rs:502-582), then the experts: one
    // upload of each input, one synchronisation at the end
    const Layer &L = h->layers[layer];
    const int E = h->cfg.num_experts, H = h->cfg.hidden_size;
    hipStream_t s = h->stream;
    const size_t lbytes = sizeof(float) * (size_t)n * (size_t)E, xbytes = sizeof(float) * (size_t)n * (size_t)H;
    if ((rc = upload_rows(h, h->logits, router_logits, lbytes, s, 0))) return rc;
    if ((rc = upload_rows(h, h->xin, xs, xbytes, s, lbytes <= kPinIO ? (lbytes + 63) / 64 * 64 : kPinIO))) return rc;
    const ExpertBanks b = banks_of(h, L);
    if (n <= 8 && n < batched_from(h, L) && is_quant_type(L.gate_type) && H % 64 == 0 && gate_up_routes_inline(b, top_k) &&
        down_combine_supported(b, top_k)) {
        // few tokens: the decode pair, gate/up routing by itself from the uploaded logits
        RouteInline route;
        route.logits = h->logits;
        route.flavour = MUMMU_ROUTER_QWEN4EXP;
        route.norm = 1;
        route.ids = h->ids;
        route.weights = h->weights;
        route.hits = L.hits;
        LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows(h->xin, (int)n, H, h->xq, s));
        LAUNCH(h, K_GATE_UP, s, launch_gate_up_routed(b, h->xq, route, (int)n, top_k, h->actq, h->flags, s));
        LAUNCH(h, K_DOWN_COMBINE, s, launch_down_combine(b, h->actq, h->ids, h->weights, (int)n, top_k, nullptr, h->xout, s));
        return download_rows(h, out, h->xout, xbytes, s, true);
    }
    LAUNCH(h, K_ROUTE_TOPK, s,
           launch_route_topk(h->logits, (int)n, E, top_k, MUMMU_ROUTER_QWEN4EXP, 1, h->ids, h->weights, L.hits, h->flags, s));
    if ((rc = run_experts(h, L, h->xin, false, n, top_k, nullptr, h->xout, s))) return rc;
    return download_rows(h, out, h->xout, xbytes, s, true);
}

int mummu_expert_run(mummu_moe *h, int layer, int expert, const float *x, int64_t rows, int hidden, float *out) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (expert < 0 || expert >= h->cfg.num_experts)
        return fail(h, MUMMU_ERR_RANGE, "expert " + std::to_string(expert) + " out of range (" + std::to_string(h->cfg.num_experts) + ")");
    if (hidden != h->cfg.hidden_size)
        return fail(h, MUMMU_ERR_SHAPE, "input hidden " + std::to_string(hidden) + " does not match expert hidden " + std::to_string(h->cfg.hidden_size));
    if (rows < 0) return fail(h, MUMMU_ERR_SHAPE, "negative row count");
    if (rows == 0) return MUMMU_OK;
    if (!x || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, rows, rows, 0))) return rc;
    hipStream_t s = h->stream;
    const size_t bytes = sizeof(float) * (size_t)rows * (size_t)hidden;
    if ((rc = upload_rows(h, h->xin, x, bytes, s))) return rc;
    ExpertBanks b = banks_of(h, h->layers[layer]);
    if (is_quant_type(b.gate_type)) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows(h->xin, (int)rows, hidden, h->xq, s));
    LAUNCH(h, K_GATE_UP, s, launch_gate_up(b, h->xin, h->xq, nullptr, (int)rows, 1, expert, h->act, h->actq, h->flags, s));
    LAUNCH(h, K_DOWN, s, launch_down(b, h->act, h->actq, nullptr, (int)rows, 1, expert, h->y, s));
    return download_rows(h, out, h->y, bytes, s, false);
}

int mummu_expert_gate_energy(mummu_moe *h, int layer, int expert, const float *x, int64_t rows, int hidden, float *energy) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (expert < 0 || expert >= h->cfg.num_experts)
        return fail(h, MUMMU_ERR_RANGE, "expert " + std::to_string(expert) + " out of range (" + std::to_string(h->cfg.num_experts) + ")");
    if (hidden != h->cfg.hidden_size)
        return fail(h, MUMMU_ERR_SHAPE, "input hidden " + std::to_string(hidden) + " does not match expert hidden " + std::to_string(h->cfg.hidden_size));
    if (rows < 0) return fail(h, MUMMU_ERR_SHAPE, "negative row count");
    if (rows == 0) return MUMMU_OK;
    if (!x || !energy) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if (hidden > 8192) return fail(h, MUMMU_ERR_SHAPE, "gate_energy: hidden above 8192 is not supported");
    if ((rc = ensure_ws(h, rows, rows, 0))) return rc;
    hipStream_t s = h->stream;
    if ((rc = upload_rows(h, h->xin, x, sizeof(float) * (size_t)rows * (size_t)hidden, s))) return rc;
    const Layer &L = h->layers[layer];
    const int I = h->cfg.expert_intermediate_size;
    const size_t n = (size_t)I * (size_t)hidden;
    const uint8_t *bank = L.gate + (size_t)expert * (size_t)I * row_bytes_of(L.gate_type, hidden);
    // scratch of this call: the gate rows as f32 (unless the bank is F32 already), the tile partials, the result
    const size_t w_floats = L.gate_type == T_F32 ? 0 : n, p_floats = (size_t)gate_energy_tiles(I) * (size_t)rows;
    float *scratch = nullptr;
    HIPCHK(h, hipMalloc(&scratch, sizeof(float) * (w_floats + p_floats + (size_t)rows)));
    float *w = w_floats ? scratch : nullptr, *partial = scratch + w_floats, *e_dev = partial + p_floats;
    hipError_t e = hipSuccess;
    if (w) e = launch_dequantize(L.gate_type, bank, n / (size_t)block_elems(L.gate_type), w, s);
    if (e == hipSuccess) e = launch_gate_energy(w ? w : (const float *)bank, h->xin, (int)rows, hidden, I, partial, e_dev, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e == hipSuccess) e = hipMemcpy(energy, e_dev, sizeof(float) * (size_t)rows, hipMemcpyDeviceToHost);
    (void)hipFree(scratch);
    if (e != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("gate_energy: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

int mummu_moe_take_hits(mummu_moe *h, int layer, uint64_t *hits) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (!hits) return fail(h, MUMMU_ERR_ARG, "null buffer");
    Layer &L = h->layers[layer];
    HIPCHK(h, hipDeviceSynchronize());
    HIPCHK(h, hipMemcpy(hits, L.hits, sizeof(uint64_t) * (size_t)h->cfg.num_experts, hipMemcpyDeviceToHost));
    HIPCHK(h, hipMemset(L.hits, 0, sizeof(uint64_t) * (size_t)h->cfg.num_experts));
    return MUMMU_OK;
}

int mummu_moe_stack_forward(mummu_moe *h, const float *x, int64_t n, int top_k, int norm, float *out, int32_t *ids) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_topk(h, top_k, h->cfg.num_experts);
    if (rc) return rc;
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (!x || !out) return fail(h, MUMMU_ERR_ARG, "null buffer");
    if ((rc = ensure_ws(h, n, n * top_k, 0))) return rc;
    const size_t bytes = sizeof(float) * (size_t)n * (size_t)h->cfg.hidden_size;
    if ((rc = upload_rows(h, h->xin, x, bytes, h->stream))) return rc;
    if ((rc = stack_impl(h, h->xin, n, top_k, norm, h->xout, h->stream, ids))) return rc;
    return download_rows(h, out, h->xout, bytes, h->stream, true);
}

int mummu_dequantize(int type, const void *bytes, size_t nbytes, float *out) {
    if (!bank_type_ok(type)) return fail(nullptr, MUMMU_ERR_TYPE, "dequant for ggml type " + std::to_string(type) + " is not implemented");
    const size_t bpb = (size_t)block_bytes(type);
    // gguf.rs:1411-1416
    if (nbytes == 0 || nbytes % bpb != 0)
        return fail(nullptr, MUMMU_ERR_BLOCKS, std::to_string(nbytes) + " bytes is not whole blocks of " + std::to_string(bpb));
    if (!bytes || !out) return fail(nullptr, MUMMU_ERR_ARG, "null buffer");
    if (mummu_device_count() < 1) return fail(nullptr, MUMMU_ERR_DEVICE, "no HIP device visible to this process");
    const size_t blocks = nbytes / bpb, n = blocks * (size_t)block_elems(type);
    uint8_t *d_in = nullptr;
    float *d_out = nullptr;
    mummu_moe *h = nullptr;
    HIPCHK(h, hipMalloc(&d_in, nbytes));
    if (hipMalloc(&d_out, n * sizeof(float)) != hipSuccess) {
        (void)hipFree(d_in);
        return fail(nullptr, MUMMU_ERR_DEVICE, "hipMalloc failed");
    }
    hipError_t e = hipMemcpy(d_in, bytes, nbytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = launch_dequantize(type, d_in, blocks, d_out, nullptr);
    if (e == hipSuccess) e = hipMemcpy(out, d_out, n * sizeof(float), hipMemcpyDeviceToHost);
    (void)hipFree(d_in);
    (void)hipFree(d_out);
    if (e != hipSuccess) return fail(nullptr, MUMMU_ERR_DEVICE, std::string("dequantize: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

int mummu_moe_dequantize_expert(mummu_moe *h, int layer, int which, int expert, float *out) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (expert < 0 || expert >= h->cfg.num_experts) return fail(h, MUMMU_ERR_RANGE, "expert out of range");
    if (which < 0 || which > 2 || !out) return fail(h, MUMMU_ERR_ARG, "which must be 0 (gate), 1 (up) or 2 (down)");
    const Layer &L = h->layers[layer];
    const int H = h->cfg.hidden_size, I = h->cfg.expert_intermediate_size;
    const int type = which == 0 ? L.gate_type : (which == 1 ? L.up_type : L.down_type);
    const int in_dim = which == 2 ? I : H, out_dim = which == 2 ? H : I;
    const uint8_t *base = which == 0 ? L.gate : (which == 1 ? L.up : L.down);
    const size_t rb = row_bytes_of(type, in_dim);
    const size_t n = (size_t)in_dim * (size_t)out_dim;
    float *d_out = nullptr;
    HIPCHK(h, hipMalloc(&d_out, n * sizeof(float)));
    hipError_t e = launch_dequantize(type, base + (size_t)expert * (size_t)out_dim * rb, n / (size_t)block_elems(type), d_out, h->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
    if (e == hipSuccess) e = hipMemcpy(out, d_out, n * sizeof(float), hipMemcpyDeviceToHost);
    (void)hipFree(d_out);
    if (e != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("dequantize_expert: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

int mummu_moe_forward_device(mummu_moe *h, int layer, const float *x_dev, int64_t n, int top_k, int norm, float *out_dev,
                             void *stream) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if ((rc = check_device_call(h, n, top_k, x_dev, out_dev))) return rc;
    if (n == 0) return MUMMU_OK;
    return forward_impl(h, layer, x_dev, n, top_k, norm, nullptr, out_dev, (hipStream_t)stream, nullptr, /*may_defer=*/true);
}

int mummu_moe_forward_device_noalloc(mummu_moe *h, int layer, const float *x_dev, int64_t n, int top_k, int norm, float *out_dev,
                                     void *stream) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if ((rc = check_topk(h, top_k, h->cfg.num_experts))) return rc;
    if (!x_dev || !out_dev) return fail(h, MUMMU_ERR_ARG, "null device pointer");
    if (((uintptr_t)x_dev & 15) || ((uintptr_t)out_dev & 15)) return fail(h, MUMMU_ERR_ARG, "device buffers must be 16-byte aligned");
    if (n < 0) return fail(h, MUMMU_ERR_SHAPE, "negative token count");
    if (n == 0) return MUMMU_OK;
    if (h->timing) return fail(h, MUMMU_ERR_ARG, "kernel timing creates events; disable it for the call that allocates nothing");
    const Layer &L = h->layers[layer];
    if (L.sh_loaded) return fail(h, MUMMU_ERR_CONFIG, "the call that allocates nothing does not serve a layer with a shared expert");
    if (n > MUMMU_NOALLOC_MAX_TOKENS || !decode_three_launches(h, L, n, top_k))
        return fail(h, n > MUMMU_NOALLOC_MAX_TOKENS ? MUMMU_ERR_TOKENS : MUMMU_ERR_CONFIG,
                    "the call that allocates nothing serves the decode form only: at most " + std::to_string(MUMMU_NOALLOC_MAX_TOKENS) +
                        " tokens, block-quantized banks, hidden a multiple of 64, top_k <= 16");
    // carve the static array: every piece starts on a 256-byte boundary
    const size_t E = (size_t)h->cfg.num_experts, H = (size_t)h->cfg.hidden_size, I = (size_t)h->cfg.expert_intermediate_size;
    const size_t nn = (size_t)n, na = nn * (size_t)top_k, xe = nn * H, ae = na * ((I + 15) / 16 * 16);
    // (the exchange state comes first: its epoch must keep its place - and its value - from call to call)
    const size_t want[] = {256, sizeof(float) * nn * E, sizeof(int32_t) * na, sizeof(float) * na,
                           xe, xe, sizeof(float) * (xe / 16), sizeof(int32_t) * (xe / 16),
                           ae, ae, sizeof(float) * (ae / 16), sizeof(int32_t) * (ae / 16), router_exchange_bytes((int)E)};
    size_t off[sizeof(want) / sizeof(want[0]) + 1] = {0};
    for (size_t i = 0; i < sizeof(want) / sizeof(want[0]); i++) off[i + 1] = (off[i] + want[i] + 255) / 256 * 256;
    const size_t need = off[sizeof(want) / sizeof(want[0])];
    if (need > MUMMU_NOALLOC_SCRATCH_BYTES)
        return fail(h, MUMMU_ERR_TOKENS, "this call needs " + std::to_string(need) + " bytes between its kernels; the static scratch holds " +
                                             std::to_string((size_t)MUMMU_NOALLOC_SCRATCH_BYTES));
    unsigned char *base = nullptr;
    if ((rc = static_scratch(h, &base))) return rc;
    DecodeScratch ws;
    ws.xstate = (unsigned long long *)(base + off[0]);
    ws.logits = (float *)(base + off[1]);
    ws.ids = (int32_t *)(base + off[2]);
    ws.weights = (float *)(base + off[3]);
    ws.xq = QAct{(int8_t *)(base + off[4]), (int8_t *)(base + off[5]), (float *)(base + off[6]), (int32_t *)(base + off[7])};
    ws.actq = QAct{(int8_t *)(base + off[8]), (int8_t *)(base + off[9]), (float *)(base + off[10]), (int32_t *)(base + off[11])};
    ws.xslots = base + off[12];
    hipStream_t s = (hipStream_t)stream;
    {
        bool done = false;
        rc = decode_two_launches(h, L, ws, x_dev, (int)n, top_k, norm, nullptr, out_dev, s, nullptr, nullptr, &done);
        if (rc || done) return rc;
    }
    // the kernels write every word of the scratch they later read; the exchange's epoch counts on from whatever the
    // array holds (it starts at zero with the process), so nothing has to be cleared between calls
    LAUNCH(h, K_ROUTER_LOGITS, s,
           launch_router_logits(x_dev, L.router, L.router_type, ws.logits, (int)n, (int)H, (int)E, ws.xq, s, nullptr, h->cfg.rms_norm_eps, nullptr));
    return decode_tail(h, L, ws, (int)n, top_k, norm, nullptr, out_dev, s);
}

int mummu_expert_run_device(mummu_moe *h, int layer, int expert, const float *x_dev, int64_t rows, int hidden, float *out_dev,
                            void *stream) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    int rc = check_layer(h, layer);
    if (rc) return rc;
    if (expert < 0 || expert >= h->cfg.num_experts)
        return fail(h, MUMMU_ERR_RANGE, "expert " + std::to_string(expert) + " out of range (" + std::to_string(h->cfg.num_experts) + ")");
    if (hidden != h->cfg.hidden_size)
        return fail(h, MUMMU_ERR_SHAPE, "input hidden " + std::to_string(hidden) + " does not match expert hidden " + std::to_string(h->cfg.hidden_size));
    if ((rc = check_device_call(h, rows, 1, x_dev, out_dev))) return rc;
    if (rows == 0) return MUMMU_OK;
    hipStream_t s = (hipStream_t)stream;
    if ((rc = flush_pending(h))) return rc;
    ExpertBanks b = banks_of(h, h->layers[layer]);
    if (is_quant_type(b.gate_type)) LAUNCH(h, K_QUANTIZE, s, launch_quantize_rows(x_dev, (int)rows, hidden, h->xq, s));
    LAUNCH(h, K_GATE_UP, s, launch_gate_up(b, x_dev, h->xq, nullptr, (int)rows, 1, expert, h->act, h->actq, h->flags, s));
    LAUNCH(h, K_DOWN, s, launch_down(b, h->act, h->actq, nullptr, (int)rows, 1, expert, out_dev, s));
    return MUMMU_OK;
}

int mummu_moe_stack_forward_device(mummu_moe *h, const float *x_dev, int64_t n, int top_k, int norm, float *out_dev, void *stream) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    int rc = check_topk(h, top_k, h->cfg.num_experts);
    if (rc) return rc;
    if ((rc = check_device_call(h, n, top_k, x_dev, out_dev))) return rc;
    if (n == 0) return MUMMU_OK;
    return stack_impl(h, x_dev, n, top_k, norm, out_dev, (hipStream_t)stream, nullptr);
}

int mummu_moe_check(mummu_moe *h, void *stream) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    const int rc = flush_pending(h);
    if (rc) return rc;
    return check_flags(h, (hipStream_t)stream);
}

int mummu_moe_last_routing(mummu_moe *h, int64_t n, int top_k, int32_t *ids, float *weights) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    if (n * top_k > h->ws_assign || n < 0 || top_k < 1) return fail(h, MUMMU_ERR_SHAPE, "routing larger than the workspace");
    const int rc = flush_pending(h);
    if (rc) return rc;
    HIPCHK(h, hipDeviceSynchronize());
    const DecodeBuffers rb = decode_buffers(h, h->routing_buf);
    if (ids) HIPCHK(h, hipMemcpy(ids, rb.ids, sizeof(int32_t) * (size_t)(n * top_k), hipMemcpyDeviceToHost));
    if (weights) HIPCHK(h, hipMemcpy(weights, rb.weights, sizeof(float) * (size_t)(n * top_k), hipMemcpyDeviceToHost));
    return MUMMU_OK;
}

void *mummu_device_alloc(size_t bytes) {
    void *p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) return nullptr;
    return p;
}

void mummu_device_free(void *p) {
    if (p) (void)hipFree(p);
}

int mummu_copy_to_device(void *dst, const void *src, size_t bytes) {
    mummu_moe *h = nullptr;
    HIPCHK(h, hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return MUMMU_OK;
}

int mummu_copy_to_host(void *dst, const void *src, size_t bytes) {
    mummu_moe *h = nullptr;
    HIPCHK(h, hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return MUMMU_OK;
}

int mummu_device_synchronize(void) {
    mummu_moe *h = nullptr;
    HIPCHK(h, hipDeviceSynchronize());
    return MUMMU_OK;
}

int mummu_device_name(char *buf, size_t len) {
    mummu_moe *h = nullptr;
    if (!buf || len == 0) return fail(nullptr, MUMMU_ERR_ARG, "null buffer");
    hipDeviceProp_t p;
    HIPCHK(h, hipGetDeviceProperties(&p, 0));
    snprintf(buf, len, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
    return MUMMU_OK;
}

void *mummu_moe_stream(mummu_moe *h) { return h ? (void *)h->stream : nullptr; }

int mummu_moe_set_router_exchange(mummu_moe *h, int enable, unsigned spin_ticks) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    h->router_exchange = enable < 0 ? 0 : (enable > 2 ? 2 : enable);
    h->spin_ticks = spin_ticks;
    return MUMMU_OK;
}

int mummu_moe_set_layer_fusion(mummu_moe *h, int enable) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    h->layer_fusion = enable < 0 ? 0 : (enable > 2 ? 2 : enable);
    return MUMMU_OK;
}

int mummu_moe_set_deferred_combine(mummu_moe *h, int enable) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    h->deferred_combine = enable != 0;
    return MUMMU_OK;
}

int mummu_moe_set_tile_order(mummu_moe *h, int enable) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    h->tile_order = enable < 0 ? -1 : (enable != 0);
    return MUMMU_OK;
}

int mummu_moe_flush(mummu_moe *h) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    return entry.rc;
}

int mummu_moe_router_exchange_state(mummu_moe *h, int *usable, uint64_t *fallbacks) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    Entry entry(h);
    if (entry.rc) return entry.rc;
    if (usable) *usable = h->router_exchange && h->xcd_round_robin;
    if (fallbacks) {
        HIPCHK(h, hipDeviceSynchronize());
        unsigned long long v = 0, zero = 0;
        HIPCHK(h, hipMemcpy(&v, h->xstate + 1, sizeof(v), hipMemcpyDeviceToHost));
        HIPCHK(h, hipMemcpy(h->xstate + 1, &zero, sizeof(zero), hipMemcpyHostToDevice));
        h->fallbacks_seen = 0;
        *fallbacks = v;
    }
    return MUMMU_OK;
}

int mummu_graph_begin(mummu_moe *h) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    if (h->timing) return fail(h, MUMMU_ERR_ARG, "kernel timing records events; disable it before capturing a graph");
    {
        Entry entry(h);  // (a sum pending from eager calls is enqueued ahead of the graph, not inside it)
        if (entry.rc) return entry.rc;
    }
    HIPCHK(h, hipStreamBeginCapture(h->stream, hipStreamCaptureModeThreadLocal));
    return MUMMU_OK;
}

int mummu_graph_end(mummu_moe *h, void **graph_exec) {
    if (!h || !graph_exec) return fail(h, MUMMU_ERR_ARG, "null argument");
    hipGraph_t g = nullptr;
    std::lock_guard<std::mutex> lock(h->mu);
    const int frc = flush_pending(h);  // the last captured step's sum becomes the graph's last node
    hipError_t ce = hipStreamEndCapture(h->stream, &g);
    if (frc) {
        if (g) (void)hipGraphDestroy(g);
        return frc;
    }
    if (ce != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("hipStreamEndCapture: ") + hipGetErrorString(ce));
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("hipGraphInstantiate: ") + hipGetErrorString(e));
    *graph_exec = (void *)new CapturedGraph{ex, h->generation};
    return MUMMU_OK;
}

// A captured graph holds raw pointers into the handle's workspace and weights: refuse to replay it once any of
// them has been freed.
static int graph_usable(mummu_moe *h, const CapturedGraph *g) {
    if (g->generation != h->generation)
        return fail(h, MUMMU_ERR_STALE, "this graph was captured before the handle's workspace grew or weights were reloaded; "
                                        "it points at freed device memory - capture it again");
    return MUMMU_OK;
}

int mummu_graph_launch(mummu_moe *h, void *graph_exec) {
    if (!h || !graph_exec) return fail(h, MUMMU_ERR_ARG, "null argument");
    const CapturedGraph *g = (const CapturedGraph *)graph_exec;
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = graph_usable(h, g);
    if (rc) return rc;
    HIPCHK(h, hipGraphLaunch(g->exec, h->stream));
    return MUMMU_OK;
}

int mummu_graph_launch_timed(mummu_moe *h, void *graph_exec, int reps, float *ms) {
    if (!h || !graph_exec || !ms) return fail(h, MUMMU_ERR_ARG, "null argument");
    if (reps < 1 || reps > 65536) return fail(h, MUMMU_ERR_ARG, "reps must be in 1..=65536");
    const CapturedGraph *g = (const CapturedGraph *)graph_exec;
    Entry entry(h);
    if (entry.rc) return entry.rc;
    int rc = graph_usable(h, g);
    if (rc) return rc;
    std::vector<hipEvent_t> ev((size_t)reps + 1, nullptr);
    hipError_t e = hipSuccess;
    for (auto &x : ev)
        if (e == hipSuccess) e = hipEventCreate(&x);
    // all replays are enqueued back to back with an event between neighbours; one synchronisation at the end
    if (e == hipSuccess) e = hipEventRecord(ev[0], h->stream);
    for (int i = 0; i < reps && e == hipSuccess; i++) {
        e = hipGraphLaunch(g->exec, h->stream);
        if (e == hipSuccess) e = hipEventRecord(ev[(size_t)i + 1], h->stream);
    }
    if (e == hipSuccess) e = hipEventSynchronize(ev[(size_t)reps]);
    for (int i = 0; i < reps && e == hipSuccess; i++) e = hipEventElapsedTime(&ms[i], ev[(size_t)i], ev[(size_t)i + 1]);
    for (auto x : ev)
        if (x) (void)hipEventDestroy(x);
    if (e != hipSuccess) return fail(h, MUMMU_ERR_DEVICE, std::string("timed graph replay: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

void mummu_graph_destroy(void *graph_exec) {
    if (!graph_exec) return;
    CapturedGraph *g = (CapturedGraph *)graph_exec;
    (void)hipGraphExecDestroy(g->exec);
    delete g;
}

int mummu_timer_start(mummu_moe *h) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    HIPCHK(h, hipEventRecord(h->t0, h->stream));
    return MUMMU_OK;
}

int mummu_timer_stop(mummu_moe *h, float *ms) {
    if (!h || !ms) return fail(h, MUMMU_ERR_ARG, "null argument");
    HIPCHK(h, hipEventRecord(h->t1, h->stream));
    HIPCHK(h, hipEventSynchronize(h->t1));
    HIPCHK(h, hipEventElapsedTime(ms, h->t0, h->t1));
    return MUMMU_OK;
}

namespace {
__global__ __launch_bounds__(256) void probe_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}
}  // namespace

int mummu_probe_copy(void *dst_dev, const void *src_dev, size_t bytes, void *stream) {
    if (!dst_dev || !src_dev || (bytes & 15) || ((uintptr_t)dst_dev & 15) || ((uintptr_t)src_dev & 15))
        return fail(nullptr, MUMMU_ERR_ARG, "probe_copy: null, unaligned or ragged buffers");
    if (bytes == 0) return MUMMU_OK;
    const size_t n16 = bytes / 16;
    const size_t want = (n16 + 255) / 256;
    const unsigned grid = (unsigned)(want < 8192 ? want : 8192);
    launch_kernel(probe_copy_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (uint4 *)dst_dev, (const uint4 *)src_dev, n16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(nullptr, MUMMU_ERR_DEVICE, std::string("probe_copy: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

extern "C++" {
namespace {
typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));
constexpr int kProbeRows = 128;   // rows a workgroup walks in the strided forms: the output slab of the grouped GEMMs

// PIECE bytes of each of the slab's rows per step, one step's loads issued and waited for before the next
// (PIECE = 0: the slab front to back, 4 KB per step).  What is read goes nowhere.
template <int PIECE>
__global__ __launch_bounds__(256) void probe_read_kernel(const uint8_t *__restrict__ src, int row_bytes) {
    const int tid = threadIdx.x;
    const uint8_t *slab = src + (size_t)blockIdx.x * kProbeRows * (size_t)row_bytes;
    probe_u32x4 acc = {0u, 0u, 0u, 0u};
    if constexpr (PIECE == 0) {
        const int steps = kProbeRows * row_bytes / 4096;
        for (int i = 0; i < steps; i++) acc ^= *(const probe_u32x4 *)(slab + (size_t)i * 4096 + tid * 16);
    } else {
        constexpr int LPR = PIECE / 16, RPP = 256 / LPR, PASSES = kProbeRows / RPP;
        const uint8_t *base = slab + (size_t)(tid / LPR) * (size_t)row_bytes + (tid % LPR) * 16;
        const int steps = row_bytes / PIECE;
        for (int st = 0; st < steps; st++) {
            probe_u32x4 r[PASSES];
#pragma unroll
            for (int p = 0; p < PASSES; p++) r[p] = *(const probe_u32x4 *)(base + (size_t)p * RPP * (size_t)row_bytes + (size_t)st * PIECE);
#pragma unroll
            for (int p = 0; p < PASSES; p++) acc ^= r[p];
        }
    }
    asm volatile("" ::"v"(acc));
}
}  // namespace
}  // extern "C++"

int mummu_probe_read(const void *src_dev, size_t bytes, int row_bytes, int piece_bytes, void *stream) {
    if (!src_dev || ((uintptr_t)src_dev & 15) || row_bytes < 128 || (row_bytes & 127))
        return fail(nullptr, MUMMU_ERR_ARG, "probe_read: null or unaligned buffer, or a row that is not a multiple of 128 bytes");
    const size_t slab = (size_t)kProbeRows * (size_t)row_bytes;
    const size_t slabs = bytes / slab;
    if (slabs == 0 || slabs > 0x7fffffffull) return fail(nullptr, MUMMU_ERR_ARG, "probe_read: fewer bytes than one slab of 128 rows");
    const dim3 grid((unsigned)slabs), block(256);
    const uint8_t *src = (const uint8_t *)src_dev;
    switch (piece_bytes) {
    case 0: launch_kernel(probe_read_kernel<0>, grid, block, 0, (hipStream_t)stream, src, row_bytes); break;
    case 32: launch_kernel(probe_read_kernel<32>, grid, block, 0, (hipStream_t)stream, src, row_bytes); break;
    case 64: launch_kernel(probe_read_kernel<64>, grid, block, 0, (hipStream_t)stream, src, row_bytes); break;
    case 128: launch_kernel(probe_read_kernel<128>, grid, block, 0, (hipStream_t)stream, src, row_bytes); break;
    default: return fail(nullptr, MUMMU_ERR_ARG, "probe_read: piece_bytes is 0 (front to back), 32, 64 or 128");
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(nullptr, MUMMU_ERR_DEVICE, std::string("probe_read: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

int mummu_moe_kernel_timing(mummu_moe *h, int enable) {
    if (!h) return fail(nullptr, MUMMU_ERR_ARG, "null handle");
    h->timing = enable != 0;
    return MUMMU_OK;
}

int mummu_moe_kernel_times(mummu_moe *h, const char **names, double *total_ms, int64_t *launches, int max_slots) {
    if (!h || !names || !total_ms || !launches) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;
    const int n = max_slots < K_SLOTS ? max_slots : (int)K_SLOTS;
    for (int i = 0; i < n; i++) {
        names[i] = kSlotNames[i];
        total_ms[i] = 0.0;
        launches[i] = 0;
    }
    for (auto &t : h->timed) {
        float ms = 0.0f;
        if (t.slot < n && hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess) {
            total_ms[t.slot] += ms;
            launches[t.slot]++;
        }
        h->event_pool.push_back(t.start);
        h->event_pool.push_back(t.stop);
    }
    h->timed.clear();
    return n;
}

}  // extern "C"
