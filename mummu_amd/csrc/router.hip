// Router of the sparse MoE block: logits GEMV, fused softmax / top-k / renormalise, and the
// pre-norm + residual helpers of the layer wrapper.
//
// Reference semantics: nn/moe.rs:139-150 (Linear, f32 softmax over all experts, top-k,
// optional renorm), models/qwen4exp/experts.rs:502-582 (the ggml-flavoured router),
// models/olmoe.rs:566-572 (x + MoE(RmsNorm(x))).
//
// Summation orders are fixed so the routing indices are reproducible bit for bit:
//   * a logit is 512 strided partial sums (element i -> partial i mod 512, one fma per
//     element in ascending i).  Lane l of the wave owns partials 8l..8l+7, folds them as
//     ((a0+a4)+(a1+a5))+((a2+a6)+(a3+a7)), and the 64 lane sums fold pairwise over adjacent
//     lanes (butterfly offsets 1,2,...,32).
//   * softmax normaliser and top-k renorm sums run sequentially in ascending expert /
//     slot order (f32, or f64 for the qwen4exp flavour), as the reference spells them out.
#include "device_utils.h"
#include "kernels.h"
#include "route_common.h"

MUMMU_TRACE_UNIT(router)

namespace mummu {

constexpr int kRouterTokensPerBlock = 4;
constexpr int kRouterChunks = 4;  // rows of up to 2048 elements take the all-loads-first form at one token

// One wave per expert row; the wave walks the row in chunks of 512 elements and serves
// kRouterTokensPerBlock tokens from each loaded weight chunk.
// NORM: x is the raw residual stream and the kernel works on RmsNorm(x) = (x * r) * gamma instead,
// r from the sum of squares in the same 512-partial order the RmsNorm kernel uses - the wave already
// holds the row in exactly that layout.  Only in the one-token form (the launcher sees to it).
template <int WT, bool VEC, bool NORM = false>
__global__ __launch_bounds__(256) void router_logits_kernel(const float *__restrict__ x, const void *__restrict__ w,
                                                            float *__restrict__ logits, int n, int hidden,
                                                            int n_experts, QAct xq, int tokens_per_block,
                                                            const float *__restrict__ gamma, float eps,
                                                            float *__restrict__ xnorm_out) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int e = blockIdx.y * (blockDim.x >> 6) + wave;
    const int t0 = blockIdx.x * tokens_per_block;  // tokens_per_block <= kRouterTokensPerBlock
    const int n_here = (n - t0) < tokens_per_block ? (n - t0) : tokens_per_block;
    // this wave's share of the activation quantization for the integer expert products:
    // 64-element slices of the tile's rows, dealt round-robin over the tile's waves
    auto quantize_share = [&](float r) {
        if (xq.hi == nullptr) return;
        const int nwaves = blockDim.x >> 6;
        const int slices_per_row = hidden / 64;  // hidden % 64 == 0 is checked by the launcher
        const int tile_tokens = n_here;
        for (int sl = blockIdx.y * nwaves + wave; sl < tile_tokens * slices_per_row; sl += gridDim.y * nwaves) {
            const int t = t0 + sl / slices_per_row;
            const int elem = (sl % slices_per_row) * 64 + lane;
            float v = x[(size_t)t * (size_t)hidden + elem];
            if (NORM) v = __fmul_rn(__fmul_rn(v, r), gamma[elem]);
            quantize_store16(v, true, xq, (size_t)t, hidden, elem);
        }
    };
    const bool one_token_fast = VEC && hidden <= 512 * kRouterChunks && n_here == 1 && e < n_experts;
    if (!one_token_fast) quantize_share(1.0f);  // (the fast form does it under its own loads, below)
    if (e >= n_experts) return;
    float acc[kRouterTokensPerBlock][8];
#pragma unroll
    for (int t = 0; t < kRouterTokensPerBlock; t++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[t][j] = 0.0f;

    const size_t wrow = (size_t)e * (size_t)hidden;
    if (one_token_fast) {
        // one token, a row of at most kRouterChunks 512-element chunks: every load of the wave is issued
        // before the first multiply (a loop would pay the memory latency once per chunk)
        float wv[kRouterChunks][8];
        float4 xa[kRouterChunks], xb[kRouterChunks];
        const float *xr = x + (size_t)t0 * (size_t)hidden;
#pragma unroll
        for (int c = 0; c < kRouterChunks; c++) {
            const int base = lane * 8 + 512 * c;
            const bool on = base < hidden;
            const int at = on ? base : 0;
            load_w8<WT>(w, wrow + (size_t)at, wv[c]);
            xa[c] = ((const float4 *)(xr + at))[0];
            xb[c] = ((const float4 *)(xr + at))[1];
        }
        float r = 1.0f;
        if (NORM) {
            float4 ga[kRouterChunks], gb[kRouterChunks];
#pragma unroll
            for (int c = 0; c < kRouterChunks; c++) {
                const int base = lane * 8 + 512 * c;
                const int at = base < hidden ? base : 0;
                ga[c] = ((const float4 *)(gamma + at))[0];
                gb[c] = ((const float4 *)(gamma + at))[1];
            }
            float a2[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < kRouterChunks; c++) {
                if (lane * 8 + 512 * c >= hidden) continue;
                const float xv[8] = {xa[c].x, xa[c].y, xa[c].z, xa[c].w, xb[c].x, xb[c].y, xb[c].z, xb[c].w};
#pragma unroll
                for (int j = 0; j < 8; j++) a2[j] = __builtin_fmaf(xv[j], xv[j], a2[j]);
            }
            float ss = __fadd_rn(__fadd_rn(__fadd_rn(a2[0], a2[4]), __fadd_rn(a2[1], a2[5])),
                                 __fadd_rn(__fadd_rn(a2[2], a2[6]), __fadd_rn(a2[3], a2[7])));
            ss = wave_sum(ss);
            r = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ss, (float)hidden), eps)));
#pragma unroll
            for (int c = 0; c < kRouterChunks; c++) {
                xa[c].x = __fmul_rn(__fmul_rn(xa[c].x, r), ga[c].x);
                xa[c].y = __fmul_rn(__fmul_rn(xa[c].y, r), ga[c].y);
                xa[c].z = __fmul_rn(__fmul_rn(xa[c].z, r), ga[c].z);
                xa[c].w = __fmul_rn(__fmul_rn(xa[c].w, r), ga[c].w);
                xb[c].x = __fmul_rn(__fmul_rn(xb[c].x, r), gb[c].x);
                xb[c].y = __fmul_rn(__fmul_rn(xb[c].y, r), gb[c].y);
                xb[c].z = __fmul_rn(__fmul_rn(xb[c].z, r), gb[c].z);
                xb[c].w = __fmul_rn(__fmul_rn(xb[c].w, r), gb[c].w);
            }
        }
        if (NORM && xnorm_out != nullptr && blockIdx.y == 0 && wave == 0) {
            // the normalised row itself, for whoever reads float activations after this launch
            float *xo = xnorm_out + (size_t)t0 * (size_t)hidden;
#pragma unroll
            for (int c = 0; c < kRouterChunks; c++) {
                const int base = lane * 8 + 512 * c;
                if (base >= hidden) continue;
                ((float4 *)(xo + base))[0] = xa[c];
                ((float4 *)(xo + base))[1] = xb[c];
            }
        }
        quantize_share(r);  // its loads join the ones above; its stores do not hold them back
#pragma unroll
        for (int c = 0; c < kRouterChunks; c++) {
            if (lane * 8 + 512 * c >= hidden) continue;  // (never adds: keeps -0 partials impossible either way)
            const float xv[8] = {xa[c].x, xa[c].y, xa[c].z, xa[c].w, xb[c].x, xb[c].y, xb[c].z, xb[c].w};
#pragma unroll
            for (int j = 0; j < 8; j++) acc[0][j] = __builtin_fmaf(xv[j], wv[c][j], acc[0][j]);
        }
    } else {
        for (int base = lane * 8; base < hidden; base += 512) {
            float wv[8];
            int cnt = hidden - base < 8 ? hidden - base : 8;
            if (VEC) {
                load_w8<WT>(w, wrow + (size_t)base, wv);
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) wv[j] = j < cnt ? load_w<WT>(w, wrow + (size_t)(base + j)) : 0.0f;
            }
#pragma unroll
            for (int t = 0; t < kRouterTokensPerBlock; t++) {
                if (t >= n_here) break;
                const float *xr = x + (size_t)(t0 + t) * (size_t)hidden + base;
                float xv[8];
                if (VEC) {
                    float4 a = ((const float4 *)xr)[0], b = ((const float4 *)xr)[1];
                    xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w; xv[4] = b.x; xv[5] = b.y; xv[6] = b.z; xv[7] = b.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 8; j++) xv[j] = j < cnt ? xr[j] : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (VEC || j < cnt) acc[t][j] = __builtin_fmaf(xv[j], wv[j], acc[t][j]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < kRouterTokensPerBlock; t++) {
        if (t >= n_here) break;
        const float *a = acc[t];
        float s = __fadd_rn(__fadd_rn(__fadd_rn(a[0], a[4]), __fadd_rn(a[1], a[5])),
                            __fadd_rn(__fadd_rn(a[2], a[6]), __fadd_rn(a[3], a[7])));
        s = wave_sum(s);
        if (lane == 0) logits[(size_t)(t0 + t) * (size_t)n_experts + (size_t)e] = s;
    }
}

bool router_logits_can_norm(const float *x, const void *w, const float *gamma, int n, int hidden) {
    return n >= 1 && n <= 8 && hidden % 64 == 0 && hidden <= 512 * kRouterChunks &&
           (((uintptr_t)x | (uintptr_t)w | (uintptr_t)gamma) & 15) == 0;
}

hipError_t launch_router_logits(const float *x, const void *w, int wtype, float *logits, int n, int hidden,
                                int n_experts, QAct xq, hipStream_t s, const float *norm_gamma, float norm_eps,
                                float *xnorm_out) {
    if (n <= 0) return hipSuccess;
    if (xq.hi != nullptr && hidden % 64 != 0) return hipErrorInvalidValue;
    if (norm_gamma && !router_logits_can_norm(x, w, norm_gamma, n, hidden)) return hipErrorInvalidValue;
    if (xnorm_out && (!norm_gamma || ((uintptr_t)xnorm_out & 15))) return hipErrorInvalidValue;
    const bool vec = (hidden % 8 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)w & 15) == 0);
    // few tokens: one wave per workgroup so the expert rows spread over as many CUs as possible
    const int waves = n <= 8 ? 1 : 4;
    // ... and one token per workgroup, which takes the all-loads-first form of the kernel
    const int tpb = n <= 8 ? 1 : kRouterTokensPerBlock;
    dim3 block(64 * waves);
    dim3 grid((n + tpb - 1) / tpb, (n_experts + waves - 1) / waves);
#define MUMMU_LAUNCH_ROUTER(WT)                                                                                       \
    do {                                                                                                              \
        if (norm_gamma)                                                                                               \
            launch_kernel(router_logits_kernel<WT, true, true>, grid, block, 0, s, x, w, logits, n, hidden, n_experts, xq, tpb, \
                          norm_gamma, norm_eps, xnorm_out);                                                           \
        else if (vec)                                                                                                 \
            launch_kernel(router_logits_kernel<WT, true>, grid, block, 0, s, x, w, logits, n, hidden, n_experts, xq, tpb, \
                          (const float *)nullptr, 0.0f, (float *)nullptr);                                                              \
        else                                                                                                          \
            launch_kernel(router_logits_kernel<WT, false>, grid, block, 0, s, x, w, logits, n, hidden, n_experts, xq, tpb, \
                          (const float *)nullptr, 0.0f, (float *)nullptr);                                                              \
    } while (0)
    switch (wtype) {
    case T_F32: MUMMU_LAUNCH_ROUTER(T_F32); break;
    case T_F16: MUMMU_LAUNCH_ROUTER(T_F16); break;
    case T_BF16: MUMMU_LAUNCH_ROUTER(T_BF16); break;
    default: return hipErrorInvalidValue;
    }
#undef MUMMU_LAUNCH_ROUTER
    return hipGetLastError();
}

constexpr int kTopkWavesPerBlock = 4;
constexpr int kMaxExperts = 64 * kMaxExpertsPerLane;

template <int JN>
__global__ __launch_bounds__(64 * kTopkWavesPerBlock) void route_topk_kernel(
    const float *__restrict__ logits, int n, int n_experts, int k, int flavour, int norm, int32_t *__restrict__ ids,
    float *__restrict__ weights, unsigned long long *__restrict__ hits, int32_t *__restrict__ flags) {
    __shared__ __attribute__((aligned(16))) RouteScratch<JN> sc[kTopkWavesPerBlock];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * kTopkWavesPerBlock + wave;
    if (t >= n) return;
    float l[JN];
#pragma unroll
    for (int j = 0; j < JN; j++) l[j] = (lane + 64 * j < n_experts) ? logits[(size_t)t * n_experts + lane + 64 * j] : 0.0f;
    route_token<JN>(l, t, n_experts, k, flavour, norm, ids, weights, hits, flags, sc[wave]);
}

hipError_t launch_route_topk(const float *logits, int n, int n_experts, int k, int flavour, int norm, int32_t *ids,
                             float *weights, unsigned long long *hits, int32_t *flags, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (n_experts > kMaxExperts || k > n_experts || k < 1) return hipErrorInvalidValue;
    dim3 block(64 * kTopkWavesPerBlock), grid((n + kTopkWavesPerBlock - 1) / kTopkWavesPerBlock);
#define MUMMU_TOPK(JN) \
    launch_kernel(route_topk_kernel<JN>, grid, block, 0, s, logits, n, n_experts, k, flavour, norm, ids, weights, hits, flags)
    if (n_experts <= 64) MUMMU_TOPK(1);
    else if (n_experts <= 128) MUMMU_TOPK(2);
    else if (n_experts <= 256) MUMMU_TOPK(4);
    else MUMMU_TOPK(8);
#undef MUMMU_TOPK
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------
// The router in ONE launch: one workgroup of 16 waves per tile of TT tokens computes every
// logit of the tile (wave w owns experts w, w+16, ...; all of a wave's weight-row loads are in
// flight before the first is used), parks them in LDS, routes the tile's tokens (one wave
// each) and quantizes the tile's activations for the integer expert products.  Nothing
// crosses a workgroup, so there is no fence, ticket or second launch on the decode path.
// ---------------------------------------------------------------------------------------
constexpr int kRouterWaves = 16;

template <int WT, bool VEC, int TT, int JN, int EPW>
__global__ __launch_bounds__(64 * kRouterWaves) void router_block_kernel(
    const float *__restrict__ x, const void *__restrict__ w, int n, int hidden, int n_experts, int k, int flavour,
    int norm, float *__restrict__ logits, int32_t *__restrict__ ids, float *__restrict__ weights,
    unsigned long long *__restrict__ hits, int32_t *__restrict__ flags, QAct xq) {
    __shared__ float s_logits[TT][64 * JN];
    __shared__ __attribute__((aligned(16))) RouteScratch<JN> sc[TT];
    MUMMU_PHASE(0);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t0 = blockIdx.x * TT;
    const int tile_tokens = (n - t0) < TT ? (n - t0) : TT;

    // EPW experts per wave: rows e = wave + 16*i
    float acc[EPW][TT][8];
#pragma unroll
    for (int i = 0; i < EPW; i++)
#pragma unroll
        for (int t = 0; t < TT; t++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[i][t][j] = 0.0f;

    for (int base = lane * 8; base < hidden; base += 512) {
        const int cnt = hidden - base < 8 ? hidden - base : 8;
        float wv[EPW][8];
#pragma unroll
        for (int i = 0; i < EPW; i++) {
            const int e = wave + kRouterWaves * i;
            const size_t wrow = (size_t)(e < n_experts ? e : 0) * (size_t)hidden;
            if (VEC) {
                load_w8<WT>(w, wrow + (size_t)base, wv[i]);
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) wv[i][j] = j < cnt ? load_w<WT>(w, wrow + (size_t)(base + j)) : 0.0f;
            }
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            if (t >= tile_tokens) break;
            const float *xr = x + (size_t)(t0 + t) * (size_t)hidden + base;
            float xv[8];
            if (VEC) {
                float4 a = ((const float4 *)xr)[0], b = ((const float4 *)xr)[1];
                xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w; xv[4] = b.x; xv[5] = b.y; xv[6] = b.z; xv[7] = b.w;
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) xv[j] = j < cnt ? xr[j] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < EPW; i++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (VEC || j < cnt) acc[i][t][j] = __builtin_fmaf(xv[j], wv[i][j], acc[i][t][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < EPW; i++) {
        const int e = wave + kRouterWaves * i;
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float *a = acc[i][t];
            float s = __fadd_rn(__fadd_rn(__fadd_rn(a[0], a[4]), __fadd_rn(a[1], a[5])),
                                __fadd_rn(__fadd_rn(a[2], a[6]), __fadd_rn(a[3], a[7])));
            s = wave_sum(s);
            if (lane == 0 && e < n_experts && t < tile_tokens) {
                s_logits[t][e] = s;
                logits[(size_t)(t0 + t) * (size_t)n_experts + (size_t)e] = s;
            }
        }
    }
    MUMMU_PHASE(1);
    // the tile's activations as 16-bit blocks: 64-element slices dealt over the waves
    if (xq.hi != nullptr) {
        const int slices_per_row = hidden / 64;  // hidden % 64 == 0 is checked by the launcher
        for (int sl = wave; sl < tile_tokens * slices_per_row; sl += kRouterWaves) {
            const int t = t0 + sl / slices_per_row;
            const int elem = (sl % slices_per_row) * 64 + lane;
            quantize_store16(x[(size_t)t * (size_t)hidden + elem], true, xq, (size_t)t, hidden, elem);
        }
    }
    __syncthreads();
    MUMMU_PHASE(2);
    if (wave < tile_tokens) {
        float l[JN];
#pragma unroll
        for (int j = 0; j < JN; j++) l[j] = (lane + 64 * j < n_experts) ? s_logits[wave][lane + 64 * j] : 0.0f;
        route_token<JN>(l, t0 + wave, n_experts, k, flavour, norm, ids, weights, hits, flags, sc[wave]);
    }
    MUMMU_PHASE(3);
}

constexpr int kRouterMaxChunks = 4;  // 512-element chunks of a row held in registers: hidden <= 2048 on the streaming path

// Streaming form (hidden = CHUNKS*512 <= 2048) for large batches: one wave owns TT tokens, keeps
// the lane's slices of their activation rows in registers (lane l owns elements 8l..8l+7 of each
// 512-chunk, i.e. partials 8l..8l+7) and walks all experts, the next weight row already in
// flight while the current one is multiplied.  The wave-wide sum leaves logit e in lane e%64, which
// is the layout the routing step wants, so nothing goes through LDS but the routing scratch and
// nothing waits on another wave.  Same summation order as router_logits_kernel.
// SPLIT > 1 (TT = 1), for batches too small to fill the chip with one wave per token: a workgroup
// of SPLIT waves per token, wave w walking experts w, w + SPLIT, ...; the logits meet in LDS and
// wave 0 routes.  The chain of dependent reductions a wave walks is SPLIT times shorter.
constexpr int kStreamWaves = 4;

template <int WT, int TT, int JN, int CHUNKS, int SPLIT = 1>
__global__ __launch_bounds__(64 * (SPLIT > 1 ? SPLIT : kStreamWaves)) void router_stream_kernel(
    const float *__restrict__ x, const void *__restrict__ w, int n, int hidden, int n_experts, int k, int flavour,
    int norm, float *__restrict__ logits, int32_t *__restrict__ ids, float *__restrict__ weights,
    unsigned long long *__restrict__ hits, int32_t *__restrict__ flags, HAct xh, QAct xq) {
    static_assert(SPLIT == 1 || TT == 1, "a split token is one token");
    __shared__ __attribute__((aligned(16))) RouteScratch<JN> sc[SPLIT > 1 ? 1 : kStreamWaves];
    __shared__ float s_logit[SPLIT > 1 ? 64 * JN : 1];
    if constexpr (SPLIT > 1) {
        // workgroups past the tokens (launched when xh or xq is set): each turns one row of x into the pairs of halfs the
        // f16-unit GEMM reads, beside the routing instead of in a launch of its own
        if ((int)blockIdx.x >= n) {
            __shared__ float s_max[SPLIT];
            const int row = (int)blockIdx.x - n;
            if (xh.hi != nullptr) {
                hact_quantize_row<64 * SPLIT>(x, hidden, xh, row, s_max);
            } else {
                // ... or into the 16-bit blocks of 16 the decode kernels read (hidden % 16 == 0: whole 16-lane rows)
                for (int e0 = threadIdx.x; e0 < hidden; e0 += 64 * SPLIT)
                    quantize_store16(x[(size_t)row * (size_t)hidden + e0], true, xq, (size_t)row, hidden, e0);
            }
            return;
        }
    }
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t0 = SPLIT > 1 ? (int)blockIdx.x : (blockIdx.x * kStreamWaves + wave) * TT;
    if (t0 >= n) return;
    constexpr int ESTEP = SPLIT > 1 ? SPLIT : 1;
    const int e_first = SPLIT > 1 ? wave : 0;
    MUMMU_PHASE(0);

    float xv[TT][CHUNKS][8];
#pragma unroll
    for (int t = 0; t < TT; t++) {
        const int tok = t0 + t < n ? t0 + t : n - 1;  // a ragged last group repeats its last token
#pragma unroll
        for (int c = 0; c < CHUNKS; c++) {
            const float4 *p = (const float4 *)(x + (size_t)tok * (size_t)hidden + c * 512 + lane * 8);
            const float4 a = p[0], b = p[1];
            xv[t][c][0] = a.x; xv[t][c][1] = a.y; xv[t][c][2] = a.z; xv[t][c][3] = a.w;
            xv[t][c][4] = b.x; xv[t][c][5] = b.y; xv[t][c][6] = b.z; xv[t][c][7] = b.w;
        }
    }
    // the lane's slice of a weight row, as stored (f32: two 16-byte words per chunk, 16-bit types: one)
    constexpr int WORDS = WT == T_F32 ? 2 : 1;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 raw[CHUNKS][WORDS], cur[CHUNKS][WORDS];
    auto fetch_row = [&](int e) {
#pragma unroll
        for (int c = 0; c < CHUNKS; c++) {
            // past the last expert the row of expert 0 is read and never used
            const size_t at = (size_t)(e < n_experts ? e : 0) * (size_t)hidden + (size_t)(c * 512 + lane * 8);
            const u32x4 *src = (const u32x4 *)((const uint8_t *)w + at * (WT == T_F32 ? 4 : 2));
#pragma unroll
            for (int i = 0; i < WORDS; i++) raw[c][i] = src[i];
        }
    };
    float l[TT][JN];
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int j = 0; j < JN; j++) l[t][j] = 0.0f;

    fetch_row(e_first);
    MUMMU_PHASE(1);
    for (int e = e_first; e < n_experts; e += ESTEP) {
        // take over the row that was in flight, start the next one, and only then touch the data:
        // the scheduling barriers keep the compiler from sinking the new loads' first use up here
#pragma unroll
        for (int c = 0; c < CHUNKS; c++)
#pragma unroll
            for (int i = 0; i < WORDS; i++) cur[c][i] = raw[c][i];
        __builtin_amdgcn_sched_barrier(0);
        fetch_row(e + ESTEP);
        __builtin_amdgcn_sched_barrier(0);
        float wv[CHUNKS][8];
#pragma unroll
        for (int c = 0; c < CHUNKS; c++) {
            if constexpr (WT == T_F32) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    wv[c][q] = __uint_as_float(cur[c][0][q]);
                    wv[c][4 + q] = __uint_as_float(cur[c][1][q]);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint16_t lo = (uint16_t)(cur[c][0][q] & 0xFFFFu), hi = (uint16_t)(cur[c][0][q] >> 16);
                    wv[c][2 * q] = WT == T_F16 ? half_bits_to_float(lo) : bf16_bits_to_float(lo);
                    wv[c][2 * q + 1] = WT == T_F16 ? half_bits_to_float(hi) : bf16_bits_to_float(hi);
                }
            }
        }
        float sum[TT];
#pragma unroll
        for (int t = 0; t < TT; t++) {
            float acc[8];
#pragma unroll
            for (int q = 0; q < 8; q++) acc[q] = 0.0f;
#pragma unroll
            for (int c = 0; c < CHUNKS; c++)
#pragma unroll
                for (int q = 0; q < 8; q++) acc[q] = __builtin_fmaf(xv[t][c][q], wv[c][q], acc[q]);
            sum[t] = __fadd_rn(__fadd_rn(__fadd_rn(acc[0], acc[4]), __fadd_rn(acc[1], acc[5])),
                               __fadd_rn(__fadd_rn(acc[2], acc[6]), __fadd_rn(acc[3], acc[7])));
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            sum[t] = wave_sum(sum[t]);
            if (SPLIT > 1) {
                if (lane == 0) s_logit[e] = sum[t];
            } else {
#pragma unroll
                for (int j = 0; j < JN; j++) l[t][j] = (e == lane + 64 * j) ? sum[t] : l[t][j];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (SPLIT > 1) {
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int j = 0; j < JN; j++) l[0][j] = (lane + 64 * j < n_experts) ? s_logit[lane + 64 * j] : 0.0f;
    }
    MUMMU_PHASE(2);
#pragma unroll
    for (int t = 0; t < TT; t++) {
        if (t0 + t >= n) break;
#pragma unroll
        for (int j = 0; j < JN; j++)
            if (lane + 64 * j < n_experts) logits[(size_t)(t0 + t) * (size_t)n_experts + lane + 64 * j] = l[t][j];
        route_token<JN>(l[t], t0 + t, n_experts, k, flavour, norm, ids, weights, hits, flags, sc[SPLIT > 1 ? 0 : wave]);
        wave_lds_sync();
    }
    MUMMU_PHASE(3);
}

template <int WT, bool VEC, int TT>
static hipError_t launch_router_block_t(const float *x, const void *w, int n, int hidden, int n_experts, int k,
                                        int flavour, int norm, float *logits, int32_t *ids, float *weights,
                                        unsigned long long *hits, int32_t *flags, QAct xq, hipStream_t s) {
    dim3 block(64 * kRouterWaves), grid((n + TT - 1) / TT);
#define MUMMU_RB(JN, EPW)                                                                                            \
    launch_kernel(router_block_kernel<WT, VEC, TT, JN, EPW>, grid, block, 0, s, x, w, n, hidden, n_experts, k, flavour, norm,   \
                                                                     logits, ids, weights, hits, flags, xq)
    if (n_experts <= 64) MUMMU_RB(1, 4);
    else if (n_experts <= 128) MUMMU_RB(2, 8);
    else return hipErrorInvalidValue;  // wider routers take the two-kernel path
#undef MUMMU_RB
    return hipGetLastError();
}

bool router_fused_supported(int n_experts) { return n_experts <= 128; }

// Which batches the router launch also converts x for: the streaming form with a workgroup per token, while those
// workgroups leave the chip room (up to 256 tokens the extra workgroups save the 4 us launch of their own: 32 / 128 /
// 256 tokens 110.6 / 119.5 / 157.0 -> 107.1 / 115.8 / 155.3 us per layer; from 512 on the router launch grows by what
// the conversion took).
bool router_converts_x(int n, int hidden, const float *x, const void *w) {
    const bool vec = (hidden % 8 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)w & 15) == 0);
    return n > 8 && n <= 256 && vec && hidden % 512 == 0 && hidden <= 512 * kRouterMaxChunks;
}

hipError_t launch_router_fused(const float *x, const void *w, int wtype, int n, int hidden, int n_experts, int k,
                               int flavour, int norm, float *logits, int32_t *ids, float *weights,
                               unsigned long long *hits, int32_t *flags, QAct xq, hipStream_t s, HAct xh) {
    if (n <= 0) return hipSuccess;
    if (xh.hi != nullptr && (xq.hi != nullptr || !router_converts_x(n, hidden, x, w))) return hipErrorInvalidValue;
    // (x quantized for the decode kernels: beside the streaming router as well where it converts x, else inside the
    // block form below)
    const bool xq_beside = xq.hi != nullptr && router_converts_x(n, hidden, x, w);
    if (n_experts > 128 || k > n_experts || k < 1) return hipErrorInvalidValue;
    if (xq.hi != nullptr && hidden % 64 != 0) return hipErrorInvalidValue;
    const bool vec = (hidden % 8 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)w & 15) == 0);
    // enough tokens to fill the chip with independent waves: activations in registers, weight
    // rows streamed (on this path the caller quantizes x separately)
    if (n > 8 && vec && (xq.hi == nullptr || xq_beside) && hidden % 512 == 0 && hidden <= 512 * kRouterMaxChunks) {
        // two tokens per wave once there are enough waves to keep every SIMD busy, else one; below a
        // wave per SIMD a token gets a whole workgroup
        const int tt = n > 2048 ? 2 : 1;
        const int split = n <= 512 ? 8 : (n <= 1024 ? 4 : (n <= 2048 ? 2 : 1));
        const int extra = (xh.hi != nullptr || xq_beside) ? n : 0;   // (split > 1 wherever router_converts_x holds)
        dim3 block(64 * kStreamWaves), grid((n + tt * kStreamWaves - 1) / (tt * kStreamWaves));
#define MUMMU_RT3(WT, JN, CH)                                                                                            \
    do {                                                                                                                 \
        if (split == 8)                                                                                                  \
            launch_kernel(router_stream_kernel<WT, 1, JN, CH, 8>, dim3(n + extra), dim3(512), 0, s, x, w, n, hidden, n_experts, k, flavour, \
                          norm, logits, ids, weights, hits, flags, xh, xq);                                                  \
        else if (split == 4)                                                                                             \
            launch_kernel(router_stream_kernel<WT, 1, JN, CH, 4>, dim3(n + extra), dim3(256), 0, s, x, w, n, hidden, n_experts, k, flavour, \
                          norm, logits, ids, weights, hits, flags, xh, xq);                                                  \
        else if (split == 2)                                                                                             \
            launch_kernel(router_stream_kernel<WT, 1, JN, CH, 2>, dim3(n + extra), dim3(128), 0, s, x, w, n, hidden, n_experts, k, flavour, \
                          norm, logits, ids, weights, hits, flags, xh, xq);                                                  \
        else if (tt == 2)                                                                                                \
            launch_kernel(router_stream_kernel<WT, 2, JN, CH>, grid, block, 0, s, x, w, n, hidden, n_experts, k, flavour, norm, \
                          logits, ids, weights, hits, flags, HAct(), QAct());                                                    \
        else                                                                                                             \
            launch_kernel(router_stream_kernel<WT, 1, JN, CH>, grid, block, 0, s, x, w, n, hidden, n_experts, k, flavour, norm, \
                          logits, ids, weights, hits, flags, HAct(), QAct());                                                    \
    } while (0)
#define MUMMU_RT2(WT, JN)                                                                                                \
    do {                                                                                                                 \
        switch (hidden / 512) {                                                                                          \
        case 1: MUMMU_RT3(WT, JN, 1); break;                                                                             \
        case 2: MUMMU_RT3(WT, JN, 2); break;                                                                             \
        case 3: MUMMU_RT3(WT, JN, 3); break;                                                                             \
        default: MUMMU_RT3(WT, JN, 4); break;                                                                            \
        }                                                                                                                \
    } while (0)
#define MUMMU_RT(WT)                                                                                                     \
    do {                                                                                                                 \
        if (n_experts <= 64) MUMMU_RT2(WT, 1);                                                                           \
        else MUMMU_RT2(WT, 2);                                                                                           \
        return hipGetLastError();                                                                                        \
    } while (0)
        switch (wtype) {
        case T_F32: MUMMU_RT(T_F32);
        case T_F16: MUMMU_RT(T_F16);
        case T_BF16: MUMMU_RT(T_BF16);
        default: return hipErrorInvalidValue;
        }
#undef MUMMU_RT
#undef MUMMU_RT2
#undef MUMMU_RT3
    }
    const bool few = n <= 64;  // few tokens: one token per workgroup
#define MUMMU_RB2(WT)                                                                                                   \
    do {                                                                                                                \
        if (few) {                                                                                                      \
            if (vec) return launch_router_block_t<WT, true, 1>(x, w, n, hidden, n_experts, k, flavour, norm, logits, ids, weights, hits, flags, xq, s); \
            return launch_router_block_t<WT, false, 1>(x, w, n, hidden, n_experts, k, flavour, norm, logits, ids, weights, hits, flags, xq, s); \
        }                                                                                                               \
        if (vec) return launch_router_block_t<WT, true, 4>(x, w, n, hidden, n_experts, k, flavour, norm, logits, ids, weights, hits, flags, xq, s); \
        return launch_router_block_t<WT, false, 4>(x, w, n, hidden, n_experts, k, flavour, norm, logits, ids, weights, hits, flags, xq, s); \
    } while (0)
    switch (wtype) {
    case T_F32: MUMMU_RB2(T_F32);
    case T_F16: MUMMU_RB2(T_F16);
    case T_BF16: MUMMU_RB2(T_BF16);
    default: return hipErrorInvalidValue;
    }
#undef MUMMU_RB2
}

// ---------------------------------------------------------------------------------------
// RmsNorm, one workgroup per token: sum of squares in the router's 512-partial order (every wave
// computes it for itself, from the same loads in the same order, so all hold the same bits), then
// (x * (1/sqrt(mean + eps))) * gamma with every step rounded separately, the row split over the
// workgroup's threads in 16-byte pieces.
// ---------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                      float eps, int hidden, float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x;
    const float *row = x + (size_t)t * (size_t)hidden;
    float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 4
    for (int base = lane * 8; base < hidden; base += 512) {
        float v[8];
        if (VEC) {  // hidden % 8 == 0: the lane's 8 elements are all inside the row
            const float4 p = *(const float4 *)(row + base), q = *(const float4 *)(row + base + 4);
            v[0] = p.x; v[1] = p.y; v[2] = p.z; v[3] = p.w; v[4] = q.x; v[5] = q.y; v[6] = q.z; v[7] = q.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = base + j < hidden ? row[base + j] : 0.0f;  // +0 leaves a partial unchanged
        }
#pragma unroll
        for (int j = 0; j < 8; j++) a[j] = __builtin_fmaf(v[j], v[j], a[j]);
    }
    float ss = __fadd_rn(__fadd_rn(__fadd_rn(a[0], a[4]), __fadd_rn(a[1], a[5])),
                         __fadd_rn(__fadd_rn(a[2], a[6]), __fadd_rn(a[3], a[7])));
    ss = wave_sum(ss);
    const float mean = __fdiv_rn(ss, (float)hidden);
    const float r = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(mean, eps)));
    float *orow = out + (size_t)t * (size_t)hidden;
    if (VEC) {
#pragma unroll 2
        for (int i = threadIdx.x * 4; i < hidden; i += 4 * blockDim.x) {
            const float4 xv = *(const float4 *)(row + i), g = *(const float4 *)(gamma + i);
            float4 o;
            o.x = __fmul_rn(__fmul_rn(xv.x, r), g.x);
            o.y = __fmul_rn(__fmul_rn(xv.y, r), g.y);
            o.z = __fmul_rn(__fmul_rn(xv.z, r), g.z);
            o.w = __fmul_rn(__fmul_rn(xv.w, r), g.w);
            *(float4 *)(orow + i) = o;
        }
    } else {
#pragma unroll 4
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) orow[i] = __fmul_rn(__fmul_rn(row[i], r), gamma[i]);
    }
}

hipError_t launch_rmsnorm(const float *x, const float *gamma, float eps, int n, int hidden, float *out, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    const bool vec = hidden % 8 == 0 && (((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)out) & 15) == 0;
    dim3 block(256), grid(n);
    if (vec) launch_kernel(rmsnorm_kernel<true>, grid, block, 0, s, x, gamma, eps, hidden, out);
    else launch_kernel(rmsnorm_kernel<false>, grid, block, 0, s, x, gamma, eps, hidden, out);
    return hipGetLastError();
}

}  // namespace mummu
