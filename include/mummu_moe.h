/*
 * mummu_moe.h - C ABI of the MI355X (gfx950) sparse mixture-of-experts block.
 *
 * One handle owns the device copy of a model's MoE blocks (router + expert banks of every
 * layer) and a pre-sized workspace.  Every entry point returns an int status (0 = ok);
 * mummu_moe_last_error() gives the message.  Nothing throws or aborts across this
 * boundary.  Host-pointer entry points borrow the caller's buffers for the call only;
 * *_device entry points take device pointers and only enqueue work on the given stream.
 *
 * Each declaration names the reference interface (physics515/Mummu, paths under
 * crates/mummu/src/) that a binding would route here.
 *
 * Weight layout at this boundary is the GGUF payload, unchanged: expert-major, row-major,
 * whole blocks per row - gate/up ne=[hidden, inter, E], down ne=[inter, hidden, E]
 * (nn/moe.rs:22-30, models/qwen4exp/experts.rs:122-136); the router is row-major
 * [E, hidden] (GGUF ffn_gate_inp, models/olmoe.rs:338-339).
 */
#ifndef MUMMU_MOE_H
#define MUMMU_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUMMU_API __attribute__((visibility("default")))

/* ggml tensor type ids (gguf.rs:298-324).  Expert banks and mummu_dequantize: all of these
 * (the block layouts of gguf.rs:1535-1797).  Router: F32, F16, BF16. */
enum mummu_ggml_type {
    MUMMU_F32 = 0,
    MUMMU_F16 = 1,
    MUMMU_Q4_0 = 2,
    MUMMU_Q4_1 = 3,
    MUMMU_Q5_0 = 6,
    MUMMU_Q5_1 = 7,
    MUMMU_Q8_0 = 8,
    MUMMU_Q4_K = 12,
    MUMMU_Q5_K = 13,
    MUMMU_Q6_K = 14,
    MUMMU_BF16 = 30
};

enum mummu_status {
    MUMMU_OK = 0,
    MUMMU_ERR_CONFIG = 1,     /* nn/moe.rs:62-76, models/olmoe.rs:210-215: E<2, k outside 1..=E, zero sizes */
    MUMMU_ERR_TYPE = 2,       /* tensor type this build has no kernel for */
    MUMMU_ERR_BLOCKS = 3,     /* a row is not whole blocks (experts.rs:150-154) / bytes not whole blocks (gguf.rs:1411-1416) */
    MUMMU_ERR_TOPK = 4,       /* top_k outside 1..=num_experts (nn/moe.rs:119-122, experts.rs:542-544) */
    MUMMU_ERR_SHAPE = 5,      /* hidden width / row count mismatch (nn/moe.rs:123-126, experts.rs:380-385) */
    MUMMU_ERR_NONFINITE = 6,  /* a router logit is inf or NaN (experts.rs:546-553) */
    MUMMU_ERR_RANGE = 7,      /* layer or expert id out of range (experts.rs:996-1007, 1112-1117) */
    MUMMU_ERR_NOT_LOADED = 8, /* the layer has no weights yet */
    MUMMU_ERR_TOKENS = 9,     /* more tokens than the workspace was sized for */
    MUMMU_ERR_DEVICE = 10,    /* no HIP device / a HIP call failed */
    MUMMU_ERR_ARG = 11,       /* null pointer or otherwise unusable argument */
    MUMMU_ERR_IO = 12,        /* a file cannot be opened, read or mapped, or ends inside its header */
    MUMMU_ERR_GGUF = 13,      /* the GGUF container breaks one of the reader's rules (gguf.rs:1226-1376) */
    MUMMU_ERR_SAFETENSORS = 14, /* a safetensors header, index or expert group breaks a rule (safetensors.rs:180-320, 600-740) */
    MUMMU_ERR_STALE = 15      /* a captured graph outlived the device buffers it points into (see mummu_graph_launch) */
};

/* Router arithmetic.  0: SparseMoe / SparseMoePerExpert (nn/moe.rs:144-150: f32 softmax,
 * top-k, weights renormalised iff norm_topk_prob).  1: qwen4exp `route`
 * (experts.rs:502-582: f64 normaliser, always renormalised with the 2^-14 floor). */
enum mummu_router_flavour { MUMMU_ROUTER_SPARSE_MOE = 0, MUMMU_ROUTER_QWEN4EXP = 1 };

/* SparseMoeConfig (nn/moe.rs:42-50) + the OlmoeConfig fields the block reads
 * (models/olmoe.rs:52-66: num_experts, num_experts_per_tok, norm_topk_prob, rms_norm_eps). */
typedef struct mummu_moe_config {
    int32_t hidden_size;
    int32_t expert_intermediate_size;
    int32_t num_experts;
    int32_t num_experts_per_tok; /* default top_k; entry points take top_k per call as the reference does */
    int32_t norm_topk_prob;
    int32_t router_flavour;      /* enum mummu_router_flavour */
    int32_t num_layers;          /* MoE blocks held by this handle (>= 1) */
    int32_t max_tokens;          /* largest b*t a call may pass; sizes the workspace */
    float rms_norm_eps;          /* used only by mummu_moe_stack_forward* */
} mummu_moe_config;

typedef struct mummu_moe mummu_moe;

/* Number of HIP devices visible to this process (0 when there is none). */
MUMMU_API int mummu_device_count(void);

/* Message of the last failure on this handle (or, for h == NULL, of the last failed call
 * that had no handle, on this thread).  Never NULL. */
MUMMU_API const char *mummu_moe_last_error(const mummu_moe *h);

/* SparseMoeConfig::init (nn/moe.rs:61-99) minus the random weights: validates the config
 * exactly as the reference asserts, then allocates the workspace on HIP device 0. */
MUMMU_API int mummu_moe_create(const mummu_moe_config *cfg, mummu_moe **out);
MUMMU_API void mummu_moe_destroy(mummu_moe *h);
/* The configuration the handle was created with (the fields of SparseMoeConfig, nn/moe.rs:42-59, plus
 * this library's own).  The file loaders below use it to refuse a model file whose geometry is not the
 * handle's before any payload is read. */
MUMMU_API int mummu_moe_get_config(const mummu_moe *h, mummu_moe_config *out);

/* The checked load of one block's tensors: `mlp.gate.weight` and
 * `mlp.experts.{gate,up,down}` <- GGUF `ffn_gate_inp`, `ffn_{gate,up,down}_exps`
 * (models/olmoe.rs:338-345; byte geometry ExpertBank::geometry, experts.rs:140-161).
 * Host pointers, GGUF payload bytes.  rms_gamma (float[hidden], may be NULL) is the
 * block's pre-norm weight (post_attention_layernorm, models/olmoe.rs:569). */
MUMMU_API int mummu_moe_load_layer(mummu_moe *h, int layer, const void *router, int router_type, const void *gate,
                                   int gate_type, const void *up, int up_type, const void *down, int down_type,
                                   const float *rms_gamma);

/* The Qwen-style block's shared expert and its sigmoid gate (models/qwen4exp/model.rs:786-804;
 * tensors `ffn_{gate,up,down}_shexp`, `ffn_gate_inp_shexp`, :228-231): once loaded, forward and
 * stack_forward of that layer return
 *     routed + shared_ffn(x) * sigmoid(<gate_vec, x>)
 * (product and sums rounded separately, in that grouping).  gate/up [inter, hidden] and down
 * [hidden, inter] in any bank type, `inter` free; gate_vec [hidden] F32 / F16 / BF16, or NULL for
 * an ungated shared expert.  The routed-only entry points (route, apply_routing, routed) are not
 * affected.  Call after mummu_moe_load_layer of the same layer. */
MUMMU_API int mummu_moe_load_shared_expert(mummu_moe *h, int layer, int inter, const void *gate, int gate_type, const void *up,
                                           int up_type, const void *down, int down_type, const void *gate_vec,
                                           int gate_vec_type);

/* The smallest token count at which a call on this layer sorts the assignments by expert and runs
 * one grouped GEMM per projection (the reference's per-expert batched form, nn/moe.rs:275-316)
 * instead of the per-token decode kernels; INT32_MAX when the layer's banks never do (or the layer is
 * not loaded).  Below it a token's result does not depend on the tokens sharing the call.  The
 * environment variable MUMMU_GEMM_MIN_TOKENS overrides the built-in crossover. */
MUMMU_API int mummu_moe_batched_from(const mummu_moe *h, int layer);

/* Bytes resident on the device for weights (ExpertExec::resident_bytes, nn/moe.rs:352). */
MUMMU_API uint64_t mummu_moe_resident_bytes(const mummu_moe *h);

/* SparseMoe::forward / SparseMoePerExpert::forward (nn/moe.rs:116, 214):
 * x [n_tokens, hidden] f32 -> out [n_tokens, hidden] f32. */
MUMMU_API int mummu_moe_forward(mummu_moe *h, int layer, const float *x, int64_t n_tokens, int top_k,
                                int norm_topk_prob, float *out);
/* The same with the activations in the caller's ambient dtype, as the reference's forward takes and returns
 * them (nn/moe.rs:116-135: the block works in f32 and the result goes back to the input's dtype): x_type
 * MUMMU_F32, MUMMU_F16 or MUMMU_BF16; x and out hold n_tokens * hidden values of that type.  16-bit rows are
 * widened exactly on the device, the f32 result is rounded to nearest even. */
MUMMU_API int mummu_moe_forward_typed(mummu_moe *h, int layer, const void *x, int x_type, int64_t n_tokens, int top_k,
                                      int norm_topk_prob, void *out);

/* SparseMoePerExpert::route (nn/moe.rs:247-290): ids/weights [n_tokens, top_k] in slot
 * (descending probability) order; logits [n_tokens, E] optional (may be NULL). */
MUMMU_API int mummu_moe_route(mummu_moe *h, int layer, const float *x, int64_t n_tokens, int top_k,
                              int norm_topk_prob, int32_t *ids, float *weights, float *logits);

/* qwen4exp `route` on caller-supplied logits (experts.rs:541-582) or the SparseMoe router
 * on them, per `flavour`.  No weights involved; n_experts is free. */
MUMMU_API int mummu_route_logits(mummu_moe *h, const float *logits, int64_t n_tokens, int n_experts, int top_k,
                                 int flavour, int norm_topk_prob, int32_t *ids, float *weights);

/* RoutedExperts::routed_moe (experts.rs:1066-1076): route these logits (qwen4exp flavour),
 * run the routed experts of `layer`, weighted sum in ascending expert id. */
MUMMU_API int mummu_moe_routed(mummu_moe *h, int layer, const float *router_logits, const float *xs, int64_t n,
                               int top_k, float *out);

/* RoutedExperts::apply_routing (experts.rs:1092-1150) == SparseMoePerExpert::run_local
 * (nn/moe.rs:296-328) == ExpertPool::run_layer (nn/moe.rs:1545-1607) for a given routing. */
MUMMU_API int mummu_moe_apply_routing(mummu_moe *h, int layer, const int32_t *ids, const float *weights,
                                      const float *xs, int64_t n, int top_k, float *out);

/* ExpertExec::run (nn/moe.rs:357) / RoutedExperts::expert_ffn (experts.rs:1015-1057):
 * SwiGLU of one expert on rows x hidden f32, row-major in and out. */
MUMMU_API int mummu_expert_run(mummu_moe *h, int layer, int expert, const float *x, int64_t rows, int hidden,
                               float *out);
/* ExpertExec::gate_energy (nn/moe.rs:411-418, DeviceExpert's at :508-521): per row of x, the sum over the
 * intermediate width of silu(x . gate_i)^2 - the gate product only, on the stored gate rows dequantized to
 * f32; the reference's skip mode compares it against a row's total (nn/moe.rs:1494-1522).  energy [rows]. */
MUMMU_API int mummu_expert_gate_energy(mummu_moe *h, int layer, int expert, const float *x, int64_t rows, int hidden,
                                       float *energy);

/* ExpertPool::take_hits (nn/moe.rs:1562-1564, 857-874): rows served per expert since the
 * last take; hits is uint64[num_experts] and the counters reset. */
MUMMU_API int mummu_moe_take_hits(mummu_moe *h, int layer, uint64_t *hits);

/* The decoder layer's MoE half for every layer of the handle, models/olmoe.rs:566-572:
 * x <- x + MoE_l(RmsNorm_l(x)), l = 0..num_layers-1.  x [n_tokens, hidden] f32 in,
 * out the final residual stream.  ids (optional) receives [num_layers, n_tokens, top_k]. */
MUMMU_API int mummu_moe_stack_forward(mummu_moe *h, const float *x, int64_t n_tokens, int top_k, int norm_topk_prob,
                                      float *out, int32_t *ids);

/* gguf::dequantize (gguf.rs:1403-1463) on the device: bytes -> f32, bit-exact.  Host
 * buffers; out holds nbytes / block_bytes * block_size floats. */
MUMMU_API int mummu_dequantize(int type, const void *bytes, size_t nbytes, float *out);

/* Dequantize one expert's matrix FROM THE DEVICE COPY held by the handle (proves the
 * resident bytes are the loaded bytes): which = 0 gate, 1 up, 2 down; out is
 * [out_dim * in_dim] f32 on the host. */
MUMMU_API int mummu_moe_dequantize_expert(mummu_moe *h, int layer, int which, int expert, float *out);

/* ---- Arithmetic of block-quantized banks, and its limit ----------------------------------------------------------
 * The reference multiplies dequantized f32 weights by f32 activations (experts.rs:401-478).  This library keeps the
 * weights packed and multiplies their integer codes by activations quantized to 16 bits per element with one f32
 * scale per block (16 consecutive elements on the decode path, 64 on the batched path): x ~ s * q, |q| <= 32512,
 * s = max|x| over the block / 32512.  Every integer sum is exact; what is lost is |x - s*q| <= s/2 per element, so
 *     |y - y_exact| <= sum over blocks of (max|x| of the block / 65024) * (sum of |w| over the block).
 * Measured as the reference measures it (error relative to the root-sum-square of the terms, experts.rs:1264-1271)
 * that is 1e-4 (Q4_K) / 6e-5 (Q8_0) on the decode path and 6e-4 / 9e-5 on the batched path for the benchmark shapes,
 * against the 2e-3 bar.  The bound is absolute per block, not relative per element: an element 2^10 below its
 * block's maximum keeps 5 bits.  This shows in one corner: a token whose SwiGLU hidden row is all but zero except
 * for one or two elements (every gate pre-activation far below zero) has outputs orders of magnitude below the
 * batch's, and relative to THAT magnitude single elements come out up to 4e-3 off (2e-8 of the batch's typical
 * output).  F32 / F16 / BF16 banks do not take this path (f32 or f16 products).
 * One exception on the batched path: Q4_K gate/up (and down) banks.  A Q4_K weight is d * (sc * q) - dmin * m
 * with sc * q < 1024 an exact half, so their grouped GEMM runs on the f16 matrix units against activations held
 * as PAIRS of halfs, x = 2^e * (hi + lo), hi = f16(x / 2^e), lo = f16(x / 2^e - hi), 2^e one power of two per row
 * (per 128 elements between the two products): 22 significant bits per element, every element of a row down to
 * 2^-24 of the row's largest.  That form measures 2e-6 by the reference's measure and has no such corner; it is
 * also the faster one.  (A row that holds an infinity comes out NaN in that form, where f32 products give an infinity.)  The environment variable MUMMU_GEMM_Q4K_F16=0, read by mummu_moe_create, keeps Q4_K on the
 * integer form above; MUMMU_GEMM_TILE_ROWS=16, 32 or 64 fixes the rows per tile of these kernels (by default the
 * library picks the form with the smallest expected cost for the batch: same results, different speed).
 * Q8_0 banks have an optional second form on the batched path, MUMMU_GEMM_Q8_F16=1 (read by mummu_moe_create):
 * the grouped GEMM of the F16 banks with every weight d * code held exactly as two halfs, x and the activations
 * between the two products rounded to halfs as for F16 / BF16 banks (values beyond 65504 overflow there).  It is
 * 1.1 to 1.5 times faster and measures 1.3e-3 to 1.6e-3 by the reference's measure where the integer form measures
 * 2e-4, which is why it is not the default; a layer with a block whose |d| * 128 is no finite half keeps the
 * integer form. */

/* ---- device-pointer entry points (no host copies, no synchronisation) ------------------
 * stream is a hipStream_t (NULL = the null stream).  Safe to capture into a HIP graph:
 * no allocation, no memset node, no host readback.  A non-finite router logit cannot be
 * reported synchronously here; mummu_moe_check() reads the flag back. */
MUMMU_API int mummu_moe_forward_device(mummu_moe *h, int layer, const float *x_dev, int64_t n_tokens, int top_k,
                                       int norm_topk_prob, float *out_dev, void *stream);
/* mummu_moe_forward_device for callers that cannot allocate device memory and do not want a workspace that was
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments, same result bits.  What its three kernels hand to one another (router logits, the
 * routing, the 16-bit activations) lives in one static device array of MUMMU_NOALLOC_SCRATCH_BYTES that every GPU
 * the library runs on holds until the process ends; the call itself calls no hipMalloc / hipFree and no allocating
 * library routine.  Limits: the decode form only - at most MUMMU_NOALLOC_MAX_TOKENS tokens, block-quantized
 * gate / up / down banks, hidden a multiple of 64, top_k <= 16, no shared expert on the layer, kernel timing off -
 * and a call whose intermediate data would not fit the array is refused (MUMMU_ERR_TOKENS / MUMMU_ERR_CONFIG, with
 * a message).  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
 * handles, two threads) race; issue them on one stream.  mummu_moe_last_routing does not see this call's routing. */
#define MUMMU_NOALLOC_SCRATCH_BYTES (4u << 20)
#define MUMMU_NOALLOC_MAX_TOKENS 8
MUMMU_API int mummu_moe_forward_device_noalloc(mummu_moe *h, int layer, const float *x_dev, int64_t n_tokens, int top_k,
                                               int norm_topk_prob, float *out_dev, void *stream);
/* A decode step of ONE token on block-quantized banks takes two launches where the device allows it: router + routing +
 * gate/up in one kernel whose workgroups pass the router logits to one another through the L2 of the XCD they share,
 * then down + combine.  No counterpart in the reference.  enable = 0: always three launches (router logits in a launch
 * of their own); 1 (default): two launches at one token; 2: two launches at every size the kernel takes (up to 8
 * tokens; slower than three from 2 tokens on).  spin_ticks bounds how long a workgroup waits for the others' logits, in
 * 10 ns units (default 5000), before it computes them itself - the result has the same bits either way, and with
 * spin_ticks = 0 no workgroup looks for the others' logits at all.  _state reports whether the two-launch form is in
 * use on this device (it is not when workgroups with equal ids modulo 8 do not share an XCD) and returns-and-clears
 * the number of workgroups that gave up waiting.  A workgroup that gives up has sat out spin_ticks first - several
 * steps' worth of time - which happens when the workgroups of a launch are not all resident at once (a device shared
 * with other work): with the default setting (1) mummu_moe_check switches the handle to three launches for good once it
 * finds 64 more of them than at its last look. */
MUMMU_API int mummu_moe_set_router_exchange(mummu_moe *h, int enable, unsigned spin_ticks);
MUMMU_API int mummu_moe_router_exchange_state(mummu_moe *h, int *usable, uint64_t *fallbacks);
/* With top_k = 8, gate / up banks of Q4_K or Q8_0, a down bank of Q4_K, Q8_0 or Q6_K, at most 128 experts and an
 * intermediate size of at most 1024, the step above can run its experts in ONE launch: the eight expert slots of a token
 * land on the eight XCDs, and the workgroups of a slot pass the expert's hidden row to one another through their XCD's L2
 * the way the router logits travel, so the down product starts inside the launch that made its input.  What is left is
 * the sum over a token's eight weighted rows, which crosses XCDs.  As a launch of its own that sum costs more than the
 * form saves (18.3 against 16.1 us per layer on the OLMoE shape), so the form pays where a later launch can take the sum
 * along: mummu_moe_set_deferred_combine.  No counterpart in the reference.  Same bits as the other forms; the same
 * spin_ticks bounds its waits, and a workgroup that gives up computes the hidden blocks it misses itself (counted by
 * _state's fallbacks).  enable = 0: never; 1 (default): in chains of deferred sums only; 2: wherever the kernel serves
 * (every decode call of up to 8 tokens when mummu_moe_set_router_exchange says 2).  Environment: MUMMU_LAYER_FUSION.
 * With at most 128 experts the launch (and the router + gate/up launch of the two-launch form) starts every slot's rows
 * on the expert whose logit has the slot's rank and confirms that pick against the routing proper while the rows are on
 * their way; a slot the routing names differently (two
 * logits whose probabilities round to the same float) is done again inside the launch: the same routing and the same
 * bits (MUMMU_EARLY_IDS=0 at mummu_moe_create: route first).  At its end the launch also reads the router of the layer after
 * its own (the first after the last: the layer a decode loop calls next) ahead, every XCD its copy, so that the next launch starts
 * on warm rows: 2 MB of extra reads per launch for 0.3 us of 14 (MUMMU_WARM_NEXT=0: not). */
MUMMU_API int mummu_moe_set_layer_fusion(mummu_moe *h, int enable);
/* enable = 1 (default 0): a mummu_moe_forward_device call that can take the one-launch form no longer enqueues the sum over
 * each token's eight weighted rows; the launch of the NEXT such call on the same stream does it on the side (a wave per
 * workgroup that would otherwise wait for the routing), so a sequence of decode steps costs one launch per step (13.7 us
 * per layer on the OLMoE shape).  out_dev of a call is then complete once the next call's work, or mummu_moe_flush, has
 * run on the stream; every other entry point of the handle, mummu_graph_begin / _end and mummu_moe_check enqueue a
 * pending sum first, so a captured graph always ends with its last step's sum and a caller that reads out_dev after
 * mummu_moe_check sees it whole.  A call whose input overlaps the pending output is preceded by that sum as well.
 * No counterpart in the reference.  Same bits as mummu_moe_forward_device without it.  Not taken with a shared expert on
 * the layer or inside mummu_moe_stack_forward*.  Environment: MUMMU_DEFERRED_COMBINE=1. */
MUMMU_API int mummu_moe_set_deferred_combine(mummu_moe *h, int enable);
/* Decode steps of several tokens on block-quantized banks can order their workgroups so that the tokens which routed to
 * the same expert read its rows through the same XCD's L2 at the same time.  The launches then fetch every distinct
 * expert once - 1.01x its bytes instead of 1.2x / 1.5x at 4 / 8 tokens of top-8 over 64 experts, where the reference
 * shares a decoded row among the rows of a call (nn/packed_gemv.rs:561-575).  From six tokens on that is also the faster
 * order (49.4 against 49.7 us per layer at 8 tokens of the OLMoE shape, 81.8 against 84.6 at 16), at two to four it
 * costs 1 - 6 %.  enable = -1 (the default): from six tokens on; 1: from two, for callers to whom the HBM traffic
 * matters more than the time; 0: never.  Same bits in every case.  Environment: MUMMU_TILE_ORDER. */
MUMMU_API int mummu_moe_set_tile_order(mummu_moe *h, int enable);
/* Enqueues the sum a deferred step left pending (nothing to do otherwise); does not synchronise. */
MUMMU_API int mummu_moe_flush(mummu_moe *h);
/* ExpertExec::run_tensor_resident (nn/moe.rs:360-371, DeviceExpert's at :470-501): the SwiGLU of one expert on rows
 * that are already on this device, the result left there; only enqueues on `stream`.  rows <= max_tokens. */
MUMMU_API int mummu_expert_run_device(mummu_moe *h, int layer, int expert, const float *x_dev, int64_t rows, int hidden,
                                      float *out_dev, void *stream);
MUMMU_API int mummu_moe_stack_forward_device(mummu_moe *h, const float *x_dev, int64_t n_tokens, int top_k,
                                             int norm_topk_prob, float *out_dev, void *stream);
/* Synchronises the stream and returns MUMMU_ERR_NONFINITE if any call since the last check
 * saw a non-finite router logit, MUMMU_ERR_DEVICE on a HIP error, else MUMMU_OK. */
MUMMU_API int mummu_moe_check(mummu_moe *h, void *stream);
/* Device copies of the last call's routing: ids int32 [n, k], weights f32 [n, k]. */
MUMMU_API int mummu_moe_last_routing(mummu_moe *h, int64_t n_tokens, int top_k, int32_t *ids, float *weights);

/* ---- GGUF container reader and expert-bank locator (host side, no device work) ----------
 * GgufFile::open / open_sharded (gguf.rs:577-714): magic, version 2 or 3, bounded counts
 * (65,536 tensors, 4,096 metadata pairs, 1 MiB strings, 2^22 array items, 4 dims, 64 shards),
 * typed metadata, `general.alignment` (a power of two, default 32), tensor table with known
 * type ids, aligned offsets, whole blocks, no duplicate names and no overlapping payloads;
 * a split set (`split.count` > 1, names `<base>-NNNNN-of-NNNNN.gguf`) is opened as one. */
typedef struct mummu_gguf mummu_gguf;

/* GgufTensorInfo (gguf.rs:403-430) plus GgufFile::payload_location (gguf.rs:1096).  Strings live as long as the
 * mummu_gguf does.  dims are in GGUF order (fastest first), padded with 1. */
typedef struct mummu_gguf_tensor {
    const char *name;
    int32_t n_dims;
    int64_t dims[4];
    int32_t ggml_type;
    int32_t shard;        /* index of the file of the split set that holds the payload */
    uint64_t file_offset; /* absolute offset in that file: its payload base + the table's offset */
    uint64_t nbytes;
    const char *path;     /* that file */
} mummu_gguf_tensor;

/* Message of the last failed mummu_gguf_* / mummu_moe_load_gguf call on this thread. */
MUMMU_API const char *mummu_gguf_last_error(void);
MUMMU_API int mummu_gguf_open(const char *path, mummu_gguf **out);
MUMMU_API void mummu_gguf_close(mummu_gguf *g);
MUMMU_API int mummu_gguf_version(const mummu_gguf *g);
MUMMU_API int64_t mummu_gguf_alignment(const mummu_gguf *g);
MUMMU_API int mummu_gguf_shard_count(const mummu_gguf *g);
MUMMU_API int mummu_gguf_tensor_count(const mummu_gguf *g);
MUMMU_API int mummu_gguf_kv_count(const mummu_gguf *g);
/* GgufFile::tensor_index (gguf.rs:1082): index of the named tensor or -1. */
MUMMU_API int mummu_gguf_find_tensor(const mummu_gguf *g, const char *name);
MUMMU_API int mummu_gguf_tensor_info(const mummu_gguf *g, int index, mummu_gguf_tensor *out);
/* The payload bytes (what GgufFile::read_tensor_f32, gguf.rs:733, reads before dequantizing),
 * mapped read-only from the owning shard; valid until close. */
MUMMU_API int mummu_gguf_tensor_data(mummu_gguf *g, int index, const void **data, uint64_t *nbytes);
/* GgufFile::get with GgufValue::as_u64 / as_f32 / as_bool / as_str (gguf.rs:140-188, 1062): typed metadata reads.
 * get_u64 takes any unsigned integer type and bool (0/1); get_f64 takes f32 and f64; get_str
 * returns NULL when the key is absent or not a string. */
MUMMU_API int mummu_gguf_get_u64(const mummu_gguf *g, const char *key, uint64_t *out);
MUMMU_API int mummu_gguf_get_f64(const mummu_gguf *g, const char *key, double *out);
MUMMU_API const char *mummu_gguf_get_str(const mummu_gguf *g, const char *key);
/* OlmoeConfig::from_gguf (models/olmoe.rs:116-179), the fields the MoE block reads, from
 * `<general.architecture>.*`: embedding_length, expert_feed_forward_length (else
 * feed_forward_length), expert_count, expert_used_count, block_count, expert_weights_norm
 * (bool, default false), attention.layer_norm_rms_epsilon (f32, required).  router_flavour is set
 * to MUMMU_ROUTER_SPARSE_MOE and max_tokens to 512; the caller may change both. */
MUMMU_API int mummu_gguf_moe_config(const mummu_gguf *g, mummu_moe_config *cfg);
/* The expert-bank locator for one layer (models/olmoe.rs:325-347, qwen4exp/experts.rs:869-911):
 * tensor indices of `blk.L.ffn_gate_inp.weight` [H,E], `blk.L.ffn_{gate,up}_exps.weight` [H,I,E],
 * `blk.L.ffn_down_exps.weight` [I,H,E] and `blk.L.ffn_norm.weight` [H] (-1 when absent), with
 * dims checked against the header's configuration, rows checked to be whole blocks and the bank
 * geometry checked against the table's byte length.  Host only. */
typedef struct mummu_gguf_moe_layer {
    int32_t router, gate, up, down, norm;
} mummu_gguf_moe_layer;
MUMMU_API int mummu_gguf_locate_moe_layer(const mummu_gguf *g, int layer, mummu_gguf_moe_layer *out);
/* RoutedExperts::open (experts.rs:869-911) + Olmoe's MoE-block load (models/olmoe.rs:338-345):
 * locates layers [first_layer, first_layer + n_layers) as above and loads them into the
 * handle's layers 0..n_layers through mummu_moe_load_layer, payload bytes unchanged (mapped
 * read-only from their shard, offsets relative to that shard's own payload base).  A layer that
 * also holds `blk.L.ffn_{gate,up,down}_shexp.weight` (2 dims) gets its shared expert loaded too,
 * gated by `blk.L.ffn_gate_inp_shexp.weight` [H] when that is present
 * (models/qwen4exp/model.rs:228-231). */
MUMMU_API int mummu_moe_load_gguf(mummu_moe *h, mummu_gguf *g, int first_layer, int n_layers);

/* ---- HF safetensors checkpoint directories (host side) -----------------------------------
 * checkpoint_shards + SafetensorsHeader::open (safetensors.rs:180-320, 377-430): a single
 * `model.safetensors` or the shards `model.safetensors.index.json` names (at most 256, each
 * checked to be on disk); every header entry checked against the payload it claims (header
 * <= 64 MiB, <= 2^20 entries, known dtype, integer dims, offsets inside the payload, shape
 * bytes == claimed bytes).  `config.json` of the same directory is parsed as OlmoeConfig. */
typedef struct mummu_st mummu_st;

/* TensorEntry (safetensors.rs:122-148) plus where its payload lies. */
typedef struct mummu_st_tensor {
    const char *name;
    const char *dtype;    /* "F32", "F16", "BF16", ... */
    int32_t n_dims;
    int64_t dims[8];      /* row-major, outermost first, padded with 1 */
    int32_t shard;
    uint64_t file_offset; /* absolute offset in that shard's file */
    uint64_t nbytes;
    const char *path;
} mummu_st_tensor;

MUMMU_API const char *mummu_st_last_error(void);
MUMMU_API int mummu_st_open(const char *dir, mummu_st **out);
MUMMU_API void mummu_st_close(mummu_st *st);
MUMMU_API int mummu_st_shard_count(const mummu_st *st);
MUMMU_API int mummu_st_tensor_count(const mummu_st *st);
MUMMU_API int mummu_st_find_tensor(const mummu_st *st, const char *name);
MUMMU_API int mummu_st_tensor_info(const mummu_st *st, int index, mummu_st_tensor *out);
/* OlmoeConfig::from_json_bytes (models/olmoe.rs:52-115, validation :180-226), the fields the MoE
 * block reads: hidden_size, intermediate_size, num_experts, num_experts_per_tok, norm_topk_prob
 * (default false), rms_norm_eps, num_hidden_layers; refuses E < 2, top-k outside 1..=E, zero
 * layers or vocab, heads that do not divide.  (Rope scaling and sliding windows belong to the
 * attention side and are not judged here.) */
MUMMU_API int mummu_olmoe_config_from_json(const char *json, size_t len, mummu_moe_config *cfg);
/* The same from the directory's config.json. */
MUMMU_API int mummu_st_moe_config(const mummu_st *st, mummu_moe_config *cfg);
/* olmoe_hf_fuse (models/olmoe.rs:405-430) as a check, no payload read: layer L has
 * `model.layers.L.mlp.gate.weight` [E,H], optional `post_attention_layernorm.weight` [H], and for
 * each of gate/up/down exactly the members `mlp.experts.{0..E-1}.*_proj.weight`, all of one float
 * dtype and of the shape the config implies (group rules of safetensors.rs:600-740). */
MUMMU_API int mummu_st_check_moe_layer(const mummu_st *st, int layer);
/* load_from_dir's fuse for the MoE block (models/olmoe.rs:432-500, safetensors.rs:450-600):
 * the members are stacked in numeric expert order into [E, out, in] banks of the source dtype
 * (BF16 / F16 / F32 kept as stored) and loaded into the handle's layers 0..n_layers. */
MUMMU_API int mummu_moe_load_safetensors(mummu_moe *h, mummu_st *st, int first_layer, int n_layers);

/* ---- the packed-GEMV custom op over burn's block-32 layout ---------------------------------
 * Q4GemvOps::q4s_gemv (nn/packed_gemv.rs:248-260; routed by try_q4s_gemv, :98-152; CubeCL kernel
 * packed_gemv_kernel, :370-451): y = x . w for a weight [K, N] stored as burn stores a quantized tensor on
 * a device (pack.rs:940-985): values two's complement in 4 bits (Q4S) or 8 bits (Q8S), element j of a u32
 * word at bits j*bits, words running along N, then one f32 scale per (k, 32 consecutive n):
 *     y[n] = sum_k float(q(k, n)) * (x[k] * scale(k, n / 32))        (two roundings per term, f32 sum).
 * A weight is uploaded once and stays in HBM; a call takes 1 row (decode) up to 64 (the reference runs a
 * short prefill row by row through the same op, :138-150).  The K split is fixed per weight shape, so a
 * call's bits do not depend on the batch or on timing. */
typedef struct mummu_packed_weight mummu_packed_weight;
/* Message of the last failed mummu_packed_* / mummu_q4s_* call on this thread. */
MUMMU_API const char *mummu_packed_last_error(void);
/* words: K * N * value_bits / 32 u32; scales: K * N / 32 f32; value_bits 4 or 8; N a multiple of 32. */
MUMMU_API int mummu_packed_weight_create(const uint32_t *words, const float *scales, int k, int n, int value_bits,
                                         mummu_packed_weight **out);
/* The same for a weight that is already in HBM (a backend's own quantized tensor): the two device buffers are
 * borrowed, not copied and not freed, and must outlive the handle. */
MUMMU_API int mummu_packed_weight_wrap_device(const uint32_t *words_dev, const float *scales_dev, int k, int n, int value_bits,
                                              mummu_packed_weight **out);
MUMMU_API void mummu_packed_weight_destroy(mummu_packed_weight *w);
/* Bytes the weight holds in HBM (values + scales: 5 bits per weight at Q4S). */
MUMMU_API uint64_t mummu_packed_weight_bytes(const mummu_packed_weight *w);
/* x [m, K] f32 -> y [m, N] f32, host pointers; m <= 64. */
MUMMU_API int mummu_q4s_gemv(mummu_packed_weight *w, const float *x, int64_t m, int k, float *y);
/* The same on device pointers; only enqueues on `stream`.  Calls on one weight must not overlap (they share
 * the partial sums of the K split). */
MUMMU_API int mummu_q4s_gemv_device(mummu_packed_weight *w, const float *x_dev, int64_t m, int k, float *y_dev, void *stream);

/* ---- plumbing for harnesses that do not link HIP themselves -----------------------------*/
MUMMU_API void *mummu_device_alloc(size_t bytes);
MUMMU_API void mummu_device_free(void *p);
MUMMU_API int mummu_copy_to_device(void *dst_dev, const void *src_host, size_t bytes);
MUMMU_API int mummu_copy_to_host(void *dst_host, const void *src_dev, size_t bytes);
MUMMU_API int mummu_device_synchronize(void);
MUMMU_API int mummu_device_name(char *buf, size_t len);

/* HIP-graph capture of whatever *_device calls are issued between begin and end on the
 * handle's own stream; launch replays it there.  No counterpart in the reference.
 *
 * A captured graph holds raw pointers into the handle's workspace and weight buffers.  The
 * *_device entry points never reallocate (they return MUMMU_ERR_TOKENS beyond max_tokens), but a
 * host-pointer call with more tokens than the workspace holds regrows it, and loading a layer or a
 * shared expert again replaces its buffers.  Either makes every graph captured before it stale:
 * mummu_graph_launch then returns MUMMU_ERR_STALE and enqueues nothing; capture the graph again.
 * graph_exec is an opaque library object (not a hipGraphExec_t); free it with mummu_graph_destroy. */
MUMMU_API void *mummu_moe_stream(mummu_moe *h);
MUMMU_API int mummu_graph_begin(mummu_moe *h);
MUMMU_API int mummu_graph_end(mummu_moe *h, void **graph_exec);
MUMMU_API int mummu_graph_launch(mummu_moe *h, void *graph_exec);
/* `reps` replays enqueued back to back, a HIP event between neighbours, one synchronisation at the
 * end: ms[i] = device milliseconds of replay i (1 <= reps <= 65536).  For benchmarks that report
 * percentiles over replays. */
MUMMU_API int mummu_graph_launch_timed(mummu_moe *h, void *graph_exec, int reps, float *ms);
MUMMU_API void mummu_graph_destroy(void *graph_exec);

/* HIP-event stopwatch on the handle's stream: elapsed milliseconds between start and stop. */
MUMMU_API int mummu_timer_start(mummu_moe *h);
MUMMU_API int mummu_timer_stop(mummu_moe *h, float *ms);

/* A plain streaming copy kernel (16 bytes per lane, grid-stride) of `bytes` bytes (a multiple
 * of 16) on the given stream: the known-size dispatch that hardware traffic counters are
 * calibrated against.  No counterpart in the reference. */
MUMMU_API int mummu_probe_copy(void *dst_dev, const void *src_dev, size_t bytes, void *stream);

/* A read-only stream over `bytes` bytes seen as rows of row_bytes bytes (a multiple of 128): one workgroup per slab
 * of 128 rows, which it reads piece_bytes (32, 64 or 128) of every row at a time, the way the grouped GEMMs walk
 * a weight slab, or front to back (piece_bytes = 0).  What is read is dropped: the launch measures what the memory
 * system delivers to a kernel that does nothing else (bench.py --probe-read).  No counterpart in the reference. */
MUMMU_API int mummu_probe_read(const void *src_dev, size_t bytes, int row_bytes, int piece_bytes, void *stream);

/* Per-kernel timing: when enabled, every kernel launched by the *_device entry points on
 * the handle's stream is bracketed by HIP events.  mummu_moe_kernel_times() synchronises and
 * returns, per kernel slot, the summed milliseconds and the launch count since the last
 * call; names[i] points at a static string.  Returns the number of slots written. */
MUMMU_API int mummu_moe_kernel_timing(mummu_moe *h, int enable);
MUMMU_API int mummu_moe_kernel_times(mummu_moe *h, const char **names, double *total_ms, int64_t *launches, int max_slots);

#ifdef __cplusplus
}
#endif
#endif /* MUMMU_MOE_H */
