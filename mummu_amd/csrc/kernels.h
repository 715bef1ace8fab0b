// Host-callable launchers of the MoE kernels.  Each returns hipGetLastError() after the
// launch; shapes are validated by the caller (moe_api.hip) before any launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "qact.h"

namespace mummu {

// error-flag words written by kernels (device int32[4])
enum : int { FLAG_NONFINITE = 0, FLAG_NONFINITE_INDEX = 1, FLAG_BAD_ID = 2 };

// dequant.hip -------------------------------------------------------------------------
// out[i] = dequantize(type, bytes)[i], bit-exact; nblocks blocks of the type.
hipError_t launch_dequantize(int type, const uint8_t *bytes, size_t nblocks, float *out, hipStream_t s);

// router.hip --------------------------------------------------------------------------
// logits[t, e] = <x[t, :], W[e, :]> in the fixed 512-partial order.  W row-major [E, H].
// xq.hi != nullptr: also the 16-bit quantization of x for the integer expert products.
// norm_gamma != nullptr (only where router_logits_can_norm says so): x is the raw residual stream and
// both outputs are computed from RmsNorm(x) = (x * r) * gamma, bit for bit what launch_rmsnorm writes;
// xnorm_out (nullable, only with norm_gamma) also receives those normalised rows.
bool router_logits_can_norm(const float *x, const void *w, const float *gamma, int n, int hidden);
hipError_t launch_router_logits(const float *x, const void *w, int wtype, float *logits, int n, int hidden,
                                int n_experts, QAct xq, hipStream_t s, const float *norm_gamma = nullptr,
                                float norm_eps = 0.0f, float *xnorm_out = nullptr);
// softmax -> top-k -> (re)normalise per token; one wave per token.
//   ids/weights [n, k] in slot order; hits (nullable) [E] += rows routed; flags see above.
hipError_t launch_route_topk(const float *logits, int n, int n_experts, int k, int flavour, int norm,
                             int32_t *ids, float *weights, unsigned long long *hits, int32_t *flags, hipStream_t s);
// Both of the above in ONE launch (num_experts <= 128), plus (xq.hi != nullptr) the 16-bit
// quantization of x for the integer expert products.
bool router_fused_supported(int n_experts);
hipError_t launch_router_fused(const float *x, const void *w, int wtype, int n, int hidden, int n_experts, int k,
                               int flavour, int norm, float *logits, int32_t *ids, float *weights,
                               unsigned long long *hits, int32_t *flags, QAct xq, hipStream_t s, HAct xh = HAct());
// xh set: the launch also writes x as pairs of halfs (only where router_converts_x holds, and never together with xq)
bool router_converts_x(int n, int hidden, const float *x, const void *w);
// x [n, D] f32 -> QAct (D % 16 == 0).
hipError_t launch_quantize_rows(const float *x, int n, int d, QAct q, hipStream_t s);
// x * rsqrt(mean(x^2) + eps) * gamma, one wave per token.
hipError_t launch_rmsnorm(const float *x, const float *gamma, float eps, int n, int hidden, float *out, hipStream_t s);

// experts.hip -------------------------------------------------------------------------
struct ExpertBanks {
    const uint8_t *gate, *up, *down;  // device, GGUF order
    int gate_type, up_type, down_type;
    int hidden, inter, n_experts;
    bool q8_half_ok = false;          // Q8_0 banks whose every |d| * 128 is inside the half range (launch_q8_scale_max)
    int tile_order_from = 6;          // decode launches of this many tokens or more: workgroups ordered so that tokens sharing an expert meet in one XCD's L2
    bool early_ids = true;            // the decode launches that route by themselves (top-8, at most 64 experts) start their rows on the eight largest logits and confirm them
};


// act[a, j] = silu(<gate_e[j,:], x_t>) * <up_e[j,:], x_t>  for assignment a = t*k + s,
// e = ids[a] (or fixed_expert >= 0 with token = a: the single-expert entry point).
// Input: xq when the gate/up banks are quantized, else x.  Output: actq when the down bank
// is quantized, else act (f32).
hipError_t launch_gate_up(const ExpertBanks &b, const float *x, QAct xq, const int32_t *ids, int n_assign, int k,
                          int fixed_expert, float *act, QAct actq, int32_t *flags, hipStream_t s);
// gate/up that routes by itself: every workgroup of token t turns the token's router logits into
// the routing (same arithmetic as route_topk, so the same bits in every workgroup) instead of
// waiting for a separate launch to publish it; the workgroup of (slot 0, row tile 0) writes
// ids / weights / hit counters for the kernels that follow.  Quantized gate/up banks feeding a
// quantized down bank, hidden <= 4096, at most 512 experts.
struct RouteInline {
    const float *logits = nullptr;  // [n, n_experts]
    int flavour = 0, norm = 0;
    int32_t *ids = nullptr;         // [n, k] out
    float *weights = nullptr;       // [n, k] out
    unsigned long long *hits = nullptr;
};
bool gate_up_routes_inline(const ExpertBanks &b, int k);
hipError_t launch_gate_up_routed(const ExpertBanks &b, QAct xq, const RouteInline &route, int n_tokens, int k, QAct actq,
                                 int32_t *flags, hipStream_t s);
// Router logits, routing and gate/up in ONE launch (the first of the two launches of a decode step): the workgroups
// of a token that share an XCD split the router's rows and pass the logits to one another through a table in that
// XCD's L2 (see gate_up_fused_kernel).  x is the block's f32 input [n, hidden]; with gamma it is the raw residual
// stream and RmsNorm(x) = (x * r) * gamma is what the block sees (xnorm_out, nullable, also receives those rows).
constexpr int kExchangeTokens = 8;  // tokens per launch the table holds
constexpr int kExchangeXcds = 16;   // the hardware id has four bits
struct RouterExchange {
    const float *x = nullptr;
    const void *w = nullptr;  // router weights [E, hidden], F32 / F16 / BF16
    int wtype = 0;
    const float *gamma = nullptr;
    float eps = 0.0f;
    float *xnorm_out = nullptr;
    void *slots = nullptr;                      // router_exchange_bytes(E) bytes, 256-byte aligned
    const unsigned long long *epoch = nullptr;  // incremented by the launch that follows (launch_down_combine)
    float *logits_out = nullptr;                // nullable [n, E]
    QAct xq_out;                                // nullable (hi == nullptr): the token rows as 16-bit blocks, for a later launch
    unsigned spin_ticks = 5000;                 // bound of the wait for the other workgroups' records, 10 ns units
    unsigned salt = 0;                          // tells launches apart that read the same epoch (a host-side launch counter)
    unsigned long long *fallbacks = nullptr;    // nullable: += 1 per workgroup that gave up waiting and computed the logits itself
};
inline size_t router_exchange_bytes(int n_experts) { return (size_t)kExchangeXcds * kExchangeTokens * (size_t)n_experts * 16; }
bool gate_up_fused_supported(const ExpertBanks &b, int k, int n_tokens, const RouterExchange &rx);
hipError_t launch_gate_up_fused(const ExpertBanks &b, const RouterExchange &rx, const RouteInline &route, int n_tokens, int k,
                                QAct actq, int32_t *flags, hipStream_t s);
// The whole expert side of a decode step in ONE launch (top_k = 8, gate/up Q4_K or Q8_0, down Q4_K / Q8_0 / Q6_K,
// inter <= 1024): the prologue of launch_gate_up_fused, gate/up, and the down product of every slot, whose hidden
// row passes between the workgroups of the XCD that owns the slot through a table in that XCD's L2 (see
// decode_layer_kernel).  Leaves y [n * k, hidden], the per-slot down sums launch_combine adds up.
constexpr int kActBlocksMax = 64;  // 16-element blocks of a hidden row the table holds (inter <= 1024)
struct LayerExchange {
    void *act_slots = nullptr;               // layer_exchange_bytes() bytes, 256-byte aligned
    float *y = nullptr;                      // [n * k, hidden] out
    unsigned long long *fallbacks = nullptr; // nullable: += 1 per workgroup that computed blocks of other workgroups itself
    // nullable: warm_bytes (a multiple of 16) that the NEXT launch will want first - the router of the layer a decode loop
    // calls next - which this launch reads ahead, through every XCD's L2, once its own rows have all been asked for
    const void *warm = nullptr;
    unsigned warm_bytes = 0;
};
// A weighted sum over the eight slots of an earlier launch's tokens that this launch performs on the side (waves that
// would otherwise wait for the routing): out = (residual +) the sum in ascending expert id, as launch_combine.
struct PendingSum {
    const float *y = nullptr;         // [n * 8, hidden]
    const int32_t *ids = nullptr;     // [n, 8]
    const float *weights = nullptr;   // [n, 8]
    const float *residual = nullptr;  // nullable [n, hidden]
    float *out = nullptr;             // [n, hidden]
    int n = 0;                        // 0: nothing pending
};
inline size_t layer_exchange_bytes() { return (size_t)kExchangeXcds * kExchangeTokens * 8 * (size_t)kActBlocksMax * 64; }
bool decode_layer_supported(const ExpertBanks &b, int k, int n_tokens, const RouterExchange &rx, const LayerExchange &lx);
hipError_t launch_decode_layer(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                               int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &pending = PendingSum());
// The same pair for float banks (F32 / F16 / BF16 gate/up and down, at most 512 experts, top_k <= 16):
// gate/up with the routing inside writes act [n*k, inter] f32, then down + combine in one launch.
bool float_decode_fused(const ExpertBanks &b, int k);
hipError_t launch_gate_up_f_routed(const ExpertBanks &b, const float *x, const RouteInline &route, int n_tokens, int k, float *act,
                                   int32_t *flags, hipStream_t s);
hipError_t launch_down_combine_f(const ExpertBanks &b, const float *act, const int32_t *ids, const float *weights, int n, int k,
                                 const float *residual, float *out, hipStream_t s);
// y[a, c] = <down_e[c,:], act[a,:]>   (actq for a quantized down bank, else act)
hipError_t launch_down(const ExpertBanks &b, const float *act, QAct actq, const int32_t *ids, int n_assign, int k,
                       int fixed_expert, float *y, hipStream_t s);
// out[t, c] = sum over the token's k slots in ASCENDING EXPERT ID of (w * y), two roundings.
// residual (nullable): out = residual + that sum.
// inv (nullable): y row of assignment a is inv[a] instead of a (dispatch-sorted layout).
// epoch_bump (nullable): the 64-bit counter of the router exchange, incremented once by this launch.
hipError_t launch_combine(const float *y, const int32_t *ids, const float *weights, const int32_t *inv, int n, int k,
                          int hidden, const float *residual, float *out, hipStream_t s, unsigned long long *epoch_bump = nullptr);
// down + combine in one launch (no y round trip): quantized down bank and top_k <= 16.
bool down_combine_supported(const ExpertBanks &b, int k);
// epoch_bump (nullable): the 64-bit counter of the router exchange, incremented once by this launch.
hipError_t launch_down_combine(const ExpertBanks &b, QAct actq, const int32_t *ids, const float *weights, int n, int k,
                               const float *residual, float *out, hipStream_t s, unsigned long long *epoch_bump = nullptr);


// out[t, :] = [residual[t, :] +] (out[t, :] + y[t, :] * sigmoid(<gate_vec, x[t, :]>)), every operation
// rounded on its own, the dot product in the router's order; gate_vec (F32 / F16 / BF16) null: no gate.
hipError_t launch_shared_add(float *out, const float *y, const float *x, const void *gate_vec, int gate_vec_type,
                             const float *residual, int n, int hidden, hipStream_t s);

// energy[t] = sum_i silu(<w_i, x_t>)^2 over the inter rows of w (f32 [inter][hidden], device); partial holds
// gate_energy_tiles(inter) * rows floats of scratch.  hidden <= 8192.
int gate_energy_tiles(int inter);
hipError_t launch_gate_energy(const float *w, const float *x, int rows, int hidden, int inter, float *partial, float *energy,
                              hipStream_t s);

// dispatch.hip ------------------------------------------------------------------------
// Stable counting sort of the assignments by expert (ranks, histograms and scans in LDS, three
// small launches): offsets[E+1], sorted[A] (position -> assignment), inv[A] (assignment ->
// position) and the grouped GEMM's work list of (expert, first position, rows <= tile_rows)
// triples.  scratch: dispatch_scratch_ints(A, E) ints.  hits (optional): per-expert row counters to
// add this batch to.
size_t dispatch_scratch_ints(int n_assign, int n_experts);
hipError_t launch_dispatch(const int32_t *ids, int n_assign, int n_experts, int tile_rows, int32_t *offsets,
                           int32_t *sorted, int32_t *inv, int32_t *tiles, int32_t *n_tiles, int32_t *scratch,
                           unsigned long long *hits, int32_t *flags, hipStream_t s);

// One expert serving rows 0..n-1 in order: sorted[i] = i and the tile list of expert 0 (tiles: 3 ints
// per tile, at least ceil(n / tile_rows) tiles).
hipError_t launch_identity_tiles(int n, int tile_rows, int32_t *sorted, int32_t *tiles, int32_t *n_tiles, hipStream_t s);

// gemm.hip ----------------------------------------------------------------------------
// Grouped GEMMs over the dispatch-sorted assignments on the matrix cores (hidden and inter
// multiples of 64): F16 and BF16 banks on the f16 units (act16: f16 [A, inter] in sorted order), F32 banks on
// the f32 units (act32: f32 [A, inter]), every
// block-quantized type on the int8 units against 16-bit activations (xq: tokens x hidden, actq:
// A x inter in sorted order; gate/up and down may differ in type).
bool grouped_gemm_supported(const ExpertBanks &b);
bool grouped_gemm_quantized(const ExpertBanks &b);
int grouped_gemm_tile_rows(const ExpertBanks &b, int n_assign, int n_experts, bool q8_half = false);
int grouped_gemm_tile_rows_q4k_f16(int n_assign, int n_experts);   // (the f16-unit Q4_K kernels: 32 or 64)
// x [n, d] f32 -> QAct64 (d % 64 == 0).
hipError_t launch_quantize_rows64(const float *x, int n, int d, QAct64 q, hipStream_t s);
// Q4_K banks can take the f16 units instead, against activations held as pairs of halfs (HAct: xh tokens x
// hidden, acth A x inter in sorted order): gate and up both Q4_K ..., ... and the down bank as well.  The
// launchers below take that form when xh.hi / acth.hi are given (pass HAct() for the int8 form); with a
// down bank of another type the gate/up launch still writes actq.
bool grouped_gemm_q4k_f16(const ExpertBanks &b);
bool grouped_gemm_q4k_f16_down(const ExpertBanks &b);
// Q8_0 banks (gate, up and down) can take the f16 kernel of the f16 banks instead: x as halfs in xh.hi alone, every
// weight as two halfs made inside the kernel, act16 between the two products.  The launchers take that form with
// q8_half set (tile rows from grouped_gemm_tile_rows(..., true): up to 128).
bool grouped_gemm_q8_f16(const ExpertBanks &b);
// max over a Q8_0 bank's blocks of |d| as half bits, folded into *max_bits (atomic max; start it at 0)
hipError_t launch_q8_scale_max(const uint8_t *bank, size_t n_blocks, uint32_t *max_bits, hipStream_t s);
// x [n, d] f32 -> HAct (d % 128 == 0).
hipError_t launch_quantize_rows_h(const float *x, int n, int d, HAct q, hipStream_t s);
// x [n, d] f32 -> halfs (d % 4 == 0): what the gate/up launch of f16 and bf16 banks reads (as xh.hi, nothing else set).
hipError_t launch_convert_rows_f16(const float *x, int n, int d, _Float16 *out, hipStream_t s);
hipError_t launch_gemm_gate_up(const ExpertBanks &b, const float *x, QAct64 xq, HAct xh, const int32_t *sorted, int k_slots,
                               const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, void *act16,
                               float *act32, QAct64 actq, HAct acth, hipStream_t s, bool q8_half = false);
hipError_t launch_gemm_down(const ExpertBanks &b, const void *act16, const float *act32, QAct64 actq, HAct acth, int n_assign,
                            const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, float *y, hipStream_t s,
                            bool q8_half = false);

}  // namespace mummu
