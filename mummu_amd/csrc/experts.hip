// SwiGLU expert products for small batches (decode): packed GEMV straight off the GGUF bytes
// resident in HBM, and the weighted combine.
//
// Reference semantics: down(silu(gate.x) * (up.x)) per routed (token, expert) pair
// (nn/moe.rs:312-316, models/qwen4exp/experts.rs:781-845), results scatter-added in
// ascending expert id with two roundings (nn/moe.rs:1590-1601, experts.rs:1137-1148).
//
// Work decomposition: blockIdx.x = one (token, expert) assignment a = t*k + s (or one token for
// the fused down+combine), blockIdx.y = a tile of output rows.  The lanes of a wave split one
// weight row in 16-byte units (Q4_K: one 16-byte slice of a super-block's nibbles; Q8_0: one
// 34-byte block; float types: consecutive elements), so every global load is a contiguous
// run, and a wave puts the loads of ALL its rows in flight before it consumes the first.
//
// Arithmetic of the quantized types (Q4_K, Q8_0): activations arrive quantized to 16-bit
// integers xq = rint(x * 32512/amax) with one f32 scale s = amax/32512 per 16 elements, split
// into two signed bytes xq = 256*hi + lo (struct QAct).  Weight codes and activation bytes
// meet in v_dot4_i32_i8, so every sum(q * xq) over 16 elements is an exact integer; only the
// scale products are floating point:
//     Q8_0 block (two halves):  d * (s0*float(sum q*xq|0) + s1*float(sum q*xq|1))
//     Q4_K sub-block pair:      d * (s0*float(sc0*sum q0*xq0) + s1*float(sc1*sum q1*xq1))
//                            - dmin * (s0*float(m0*sum xq0) + s1*float(m1*sum xq1))
// A 16-bit activation is ~2^-15 of its block maximum - about 100x finer than the int8
// activations llama.cpp multiplies these formats with - and, being a function of the token's
// own row only, keeps the result independent of how many tokens share the call.
// Float weight types (F32/F16/BF16) run an f32 fma chain per lane on the exact f32 value of
// each weight and the f32 activation.
#include "device_utils.h"
#include "kernels.h"
#include "gemv_common.h"
#include "route_common.h"
#include "decode_parts.h"

#include <algorithm>
#include <cstdint>
#include <type_traits>

MUMMU_TRACE_UNIT(experts)

namespace mummu {

constexpr int kGemvWaves = 4;  // waves per workgroup of the float kernels

// Calls f(std::integral_constant<int, TYPE>) for a bank type this file has kernels for.
template <typename F>
static hipError_t with_bank_type(int type, F &&f) {
#define MUMMU_TYPE_CASE(T) case T: return f(std::integral_constant<int, T>())
    switch (type) {
        MUMMU_TYPE_CASE(T_F32);
        MUMMU_TYPE_CASE(T_F16);
        MUMMU_TYPE_CASE(T_BF16);
        MUMMU_TYPE_CASE(T_Q8_0);
        MUMMU_TYPE_CASE(T_Q4_K);
        MUMMU_TYPE_CASE(T_Q4_0);
        MUMMU_TYPE_CASE(T_Q4_1);
        MUMMU_TYPE_CASE(T_Q5_0);
        MUMMU_TYPE_CASE(T_Q5_1);
        MUMMU_TYPE_CASE(T_Q5_K);
        MUMMU_TYPE_CASE(T_Q6_K);
    default: return hipErrorInvalidValue;
    }
#undef MUMMU_TYPE_CASE
}

// Several tokens per step (ExpertBanks::tile_order_from and up): tokens that routed to the same expert read the same
// weight rows, and the eight XCDs each have an L2 of their own, so the second read only hits if both workgroups sit
// on one XCD at about the same time.  Workgroups go to the XCDs round-robin by linear index; with grid = (kXcds,
// slots * tokens, ceil(tiles / kXcds)) the XCD is the row tile modulo 8 and every (token, slot) pair of a tile follows
// its neighbour onto that XCD: whoever shares an expert shares the lines while they are in that L2 (or on their way
// into it).  The launches then fetch the bytes of the distinct experts once (1.01x against 1.5x at eight tokens of
// top-8 over 64 experts); from six tokens on that is the faster order as well (81.8 against 84.6 us per layer at 16
// tokens), at two to four it takes 1 - 6 % more time (an XCD no longer walks through one expert's matrix from end to
// end), so by default it starts at six.  A variant of the kernels compiled for it: the plain order keeps its code.
constexpr int kXcds = 8;

// The grid of that order for `pairs` = tokens (x slots) per row tile, or false: the plain grid (not asked for, one
// token, or an extent past the limit of a grid).  x = row tile modulo 8, y = the (token, slot) pair, z = row tile / 8.
static bool tile_order_grid(bool wanted, int tokens, int pairs, int tiles, dim3 &grid) {
    const int z = (tiles + kXcds - 1) / kXcds;
    if (!wanted || tokens <= 1 || pairs > 65535 || z > 65535) return false;
    grid = dim3(kXcds, (unsigned)pairs, (unsigned)z);
    return true;
}

// ------------------------------------------------------------------------------------------
// gate/up, quantized banks: NIT iterations of rows_per_it rows per wave; the workgroup's
// rows_per_block = waves*NIT*rows_per_it output rows are a whole number of 16-element
// activation blocks, quantized for the down projection in the epilogue.
// ------------------------------------------------------------------------------------------
// RJN > 0: the kernel routes by itself, RJN experts per lane of the routing wave (see RouteInline).
template <int WT, int UPL, int NIT, bool ACTQ, int RJN = 0, bool ORDERED = false>
__global__ __launch_bounds__(1024) void gate_up_q_kernel(const uint8_t *__restrict__ gate,
                                                         const uint8_t *__restrict__ up, QAct xq,
                                                         const int32_t *__restrict__ ids, int k, int fixed_expert,
                                                         int hidden, int inter, int n_experts,
                                                         float *__restrict__ act, QAct actq,
                                                         int32_t *__restrict__ flags, RouteInline route) {
    constexpr bool ROUTE = RJN > 0;
    constexpr int JN = ROUTE ? RJN : 1;
    extern __shared__ float s_act[];  // rows_per_block floats
    __shared__ __attribute__((aligned(16))) RouteScratch<JN> s_route;
    __shared__ int s_ids[64];
    __shared__ float s_w[64];
    MUMMU_PHASE(0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // grid = (slot, row tile, token), or ORDERED: (row tile modulo 8, token * k + slot, row tile / 8)
    int slot = blockIdx.x, tile = blockIdx.y, t = blockIdx.z, slots = gridDim.x;
    if constexpr (ORDERED) {
        slots = k;
        slot = blockIdx.y % k;
        t = blockIdx.y / k;
        tile = blockIdx.z * kXcds + blockIdx.x;
        const int rows_per_block = NIT * (64 >> row_split(hidden).group_log2) * (blockDim.x >> 6);
        if (tile * rows_per_block >= inter) return;  // (the eight columns cover a whole number of tiles or a few more)
    }
    const int a = t * slots + slot;
    const RowSplit rs = row_split(hidden);
    const int unit0 = lane & (rs.group - 1);
    LaneAct<UPL> la;  // the token's activations do not depend on the routing: fetch them first
    load_lane_act<WT, UPL>(xq, (size_t)t, hidden, unit0, rs.units, la);
    if (ROUTE) {
        // wave 0 routes token t from its logits; everybody else already has the activations coming
        if (wave == 0) {
            float l[JN];
#pragma unroll
            for (int j = 0; j < JN; j++) l[j] = lane + 64 * j < n_experts ? route.logits[(size_t)t * n_experts + lane + 64 * j] : 0.0f;
            route_token<JN, false>(l, t, n_experts, k, route.flavour, route.norm, s_ids, s_w, nullptr, flags, s_route, 0);
            wave_lds_sync();
            if (slot == 0 && tile == 0 && lane < k) {
                const int id = s_ids[lane];
                route.ids[(size_t)t * k + lane] = id;
                route.weights[(size_t)t * k + lane] = s_w[lane];
                if (route.hits && (unsigned)id < (unsigned)n_experts) atomicAdd(&route.hits[id], 1ULL);
            }
            MUMMU_PHASE(6);
        }
        __syncthreads();
        MUMMU_PHASE(7);
    }
    const int e = ROUTE ? s_ids[slot] : (fixed_expert >= 0 ? fixed_expert : ids[a]);
    if ((unsigned)e >= (unsigned)n_experts) {
        if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
        return;
    }
    gate_up_tile<WT, UPL, NIT, ACTQ>(gate, up, e, a, la, rs, hidden, inter, act, actq, s_act, tile);
}

// ------------------------------------------------------------------------------------------
// Decode, first of two launches: router logits, routing and gate/up in ONE kernel.
//
// The grid is the gate/up grid (slot, row tile, token).  The prologue (decode_route_prologue: the workgroups of a
// token that share an XCD split the router's rows, pass the logits to one another through that XCD's L2, route, and
// leave the token's 16-bit row in LDS) is followed by the workgroup's tile of gate/up rows.  The epoch of the
// exchange is incremented by the launch after this one (down_combine).
// hidden <= 2048 and a multiple of 64; (slots * row tiles) a multiple of 8.
// EARLY (k = 8, at most two experts per routing lane): the rows start on the expert whose logit has the slot's rank; wave 0 confirms
// the pick behind its first row loads and a slot the routing names differently is done again (see decode_route_prologue).
// ------------------------------------------------------------------------------------------
template <int WT, int NIT, int RJN, bool EARLY>
__global__ __launch_bounds__(256) void gate_up_fused_kernel(const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up, int k,
                                                            int hidden, int inter, int n_experts, QAct actq,
                                                            int32_t *__restrict__ flags, RouteInline route, RouterExchange rx) {
    extern __shared__ float s_dyn[];  // [rows_per_block] gate/up results, then the token's 16-bit row
    __shared__ __attribute__((aligned(16))) DecodeShared<RJN> sh;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.z;  // grid = (slot, row tile, token)
    const int a = t * gridDim.x + blockIdx.x;
    const RowSplit rs = row_split(hidden);
    const int unit0 = lane & (rs.group - 1);
    const int rows_per_block = NIT * rs.rows_per_it * (blockDim.x >> 6);
    float *s_act = s_dyn;
    int8_t *s_xhi = (int8_t *)(s_dyn + rows_per_block);
    int8_t *s_xlo = s_xhi + hidden;
    float *s_xscale = (float *)(s_xlo + hidden);
    int *s_xsum = (int *)(s_xscale + hidden / 16);
    MUMMU_PHASE(0);
    RouteCarry<RJN> carry;
    decode_route_prologue<RJN, NoHook, EARLY>(k, hidden, n_experts, flags, route, rx, sh, s_xhi, s_xlo, s_xscale, s_xsum, NoHook(), &carry);
    LaneAct<1> la;
    load_lane_act_lds<WT>(s_xhi, s_xlo, s_xscale, s_xsum, unit0, rs.units, la);
    MUMMU_PHASE(14);
    int e = EARLY ? sh.early_ids[blockIdx.x] : sh.ids[blockIdx.x];
    if ((unsigned)e >= (unsigned)n_experts) {
        if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
        return;
    }
    if constexpr (EARLY) {
        auto route_rest = [&]() {
            if (wave == 0) decode_route_finish<RJN, true>(carry.l, k, n_experts, flags, route, rx, sh);
        };
        gate_up_tile<WT, 1, NIT, true, true, NoHook, NIT - 1, decltype(route_rest)>(gate, up, e, a, la, rs, hidden, inter, nullptr, actq, s_act,
                                                                                    blockIdx.y, NoHook(), route_rest);
        __syncthreads();
        if (sh.ids[blockIdx.x] != e) {  // (the same finding in every workgroup of the slot: its rows again, for the expert the routing names)
            e = sh.ids[blockIdx.x];
            if ((unsigned)e >= (unsigned)n_experts) {
                if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
                return;
            }
            gate_up_tile<WT, 1, NIT, true>(gate, up, e, a, la, rs, hidden, inter, nullptr, actq, s_act, blockIdx.y);
        }
    } else {
        gate_up_tile<WT, 1, NIT, true>(gate, up, e, a, la, rs, hidden, inter, nullptr, actq, s_act, blockIdx.y);
    }
}

// gate/up, float banks.  RJN > 0: the kernel routes by itself (see RouteInline), RJN experts per lane
// of the routing wave.
template <int WT, int VEC, int RJN = 0>
__global__ __launch_bounds__(64 * kGemvWaves) void gate_up_f_kernel(
    const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up, const float *__restrict__ x,
    const int32_t *__restrict__ ids, int k, int fixed_expert, int hidden, int inter, int n_experts,
    int rows_per_wave, float *__restrict__ act, int32_t *__restrict__ flags, RouteInline route) {
    constexpr bool ROUTE = RJN > 0;
    constexpr int JN = ROUTE ? RJN : 1;
    __shared__ __attribute__((aligned(16))) RouteScratch<JN> s_route;
    __shared__ int s_ids[64];
    __shared__ float s_w[64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.z;  // grid = (slot, row tile, token)
    const int a = t * gridDim.x + blockIdx.x;
    if (ROUTE) {
        if (wave == 0) {
            float l[JN];
#pragma unroll
            for (int j = 0; j < JN; j++) l[j] = lane + 64 * j < n_experts ? route.logits[(size_t)t * n_experts + lane + 64 * j] : 0.0f;
            route_token<JN, false>(l, t, n_experts, k, route.flavour, route.norm, s_ids, s_w, nullptr, flags, s_route, 0);
            wave_lds_sync();
            if (blockIdx.x == 0 && blockIdx.y == 0 && lane < k) {
                const int id = s_ids[lane];
                route.ids[(size_t)t * k + lane] = id;
                route.weights[(size_t)t * k + lane] = s_w[lane];
                if (route.hits && (unsigned)id < (unsigned)n_experts) atomicAdd(&route.hits[id], 1ULL);
            }
        }
        __syncthreads();
    }
    const int e = ROUTE ? s_ids[blockIdx.x] : (fixed_expert >= 0 ? fixed_expert : ids[a]);
    if ((unsigned)e >= (unsigned)n_experts) {
        if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
        return;
    }
    const size_t row_bytes = type_row_bytes(WT, hidden);
    const uint8_t *ge = gate + (size_t)e * (size_t)inter * row_bytes;
    const uint8_t *ue = up + (size_t)e * (size_t)inter * row_bytes;
    const float *xrow = x + (size_t)t * (size_t)hidden;
    float *arow = act + (size_t)a * (size_t)inter;
    const int row0 = (blockIdx.y * kGemvWaves + wave) * rows_per_wave;
    // four rows of either matrix at a time (rows_per_wave is a multiple of 4): eight loads in flight per
    // iteration; rows past the bank's end stand in for its last row and are not stored
    for (int r = 0; r < rows_per_wave; r += 4) {
        if (row0 + r >= inter) break;
        const uint8_t *rowp[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int row = row0 + r + j < inter ? row0 + r + j : inter - 1;
            rowp[j] = ge + (size_t)row * row_bytes;
            rowp[4 + j] = ue + (size_t)row * row_bytes;
        }
        float p[8];
        rows_partial_f<WT, VEC, 8>(rowp, xrow, hidden, lane, p);
#pragma unroll
        for (int j = 0; j < 8; j++) p[j] = wave_sum(p[j]);
        if (lane < 4 && row0 + r + lane < inter) {
            const float pg = lane == 0 ? p[0] : (lane == 1 ? p[1] : (lane == 2 ? p[2] : p[3]));
            const float pu = lane == 0 ? p[4] : (lane == 1 ? p[5] : (lane == 2 ? p[6] : p[7]));
            arow[row0 + r + lane] = __fmul_rn(det_silu(pg), pu);
        }
    }
}

// x [n, d] f32 -> QAct: one lane per element, 16-lane rows are the activation blocks.
__global__ __launch_bounds__(256) void quantize_rows_kernel(const float *__restrict__ x, int n, int d, QAct q) {
    const size_t total = (size_t)n * (size_t)d;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool on = i < total;  // d % 16 == 0: whole 16-lane rows are on or off together
    const size_t row = on ? i / (size_t)d : 0;
    const int elem = on ? (int)(i % (size_t)d) : 0;
    quantize_store16(on ? x[i] : 0.0f, on, q, row, d, elem);
}

hipError_t launch_quantize_rows(const float *x, int n, int d, QAct q, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (d % 16) return hipErrorInvalidValue;
    const size_t total = (size_t)n * (size_t)d;
    launch_kernel(quantize_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, x, n, d, q);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// down: y[a, c] = <down_e[c], act[a]>
// ------------------------------------------------------------------------------------------
template <int WT, int UPL, int NIT>
__global__ __launch_bounds__(64 * kGemvWaves) void down_q_kernel(const uint8_t *__restrict__ down, QAct actq,
                                                                 const int32_t *__restrict__ ids, int fixed_expert,
                                                                 int hidden, int inter, int n_experts,
                                                                 float *__restrict__ y) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = blockIdx.z * gridDim.x + blockIdx.x;  // grid = (slot, row tile, token)
    const int e = fixed_expert >= 0 ? fixed_expert : ids[a];
    if ((unsigned)e >= (unsigned)n_experts) return;  // flagged by gate_up
    const RowSplit rs = row_split(inter);
    const int sub = lane >> rs.group_log2, unit0 = lane & (rs.group - 1);
    const int rows_per_wave = NIT * rs.rows_per_it;
    const int row0 = (blockIdx.y * kGemvWaves + wave) * rows_per_wave;
    const uint32_t row_bytes = (uint32_t)type_row_bytes(WT, inter);
    const uint8_t *de = down + (size_t)uniform_index(e) * (size_t)hidden * row_bytes;  // (e is the same in every lane)
    float *yrow = y + (size_t)a * (size_t)hidden;

    RawRow<WT, UPL> rd[NIT];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int row = row0 + i * rs.rows_per_it + sub;
        const bool ok = row < hidden;
        load_row<WT, UPL>(de, (uint32_t)(ok ? row : 0) * row_bytes, unit0, rs.units, ok, rd[i]);
    }
    LaneAct<UPL> la;
    load_lane_act<WT, UPL>(actq, (size_t)a, inter, unit0, rs.units, la);
    float part[NIT];
#pragma unroll
    for (int i = 0; i < NIT; i++) part[i] = dot_row<WT, UPL>(rd[i], unit0, la);
    dispatch_group(rs.group, [&](auto group_tag) {
        constexpr int GROUP = decltype(group_tag)::value;
        const int offset = reduce_partials<NIT, GROUP>(part, lane);
        constexpr int count = reduced_count<NIT, GROUP>();
        constexpr int width = GROUP < 16 ? GROUP : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < count; j++) {
                const int row = row0 + (offset + j) * rs.rows_per_it + sub;
                if (row < hidden) yrow[row] = part[j];
            }
        }
    });
}

template <int WT, int VEC>
__global__ __launch_bounds__(64 * kGemvWaves) void down_f_kernel(const uint8_t *__restrict__ down,
                                                                 const float *__restrict__ act,
                                                                 const int32_t *__restrict__ ids, int fixed_expert,
                                                                 int hidden, int inter, int n_experts, int rows_per_wave,
                                                                 float *__restrict__ y) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = blockIdx.z * gridDim.x + blockIdx.x;  // grid = (slot, row tile, token)
    const int e = fixed_expert >= 0 ? fixed_expert : ids[a];
    if ((unsigned)e >= (unsigned)n_experts) return;
    const size_t row_bytes = type_row_bytes(WT, inter);
    const uint8_t *de = down + (size_t)e * (size_t)hidden * row_bytes;
    const float *arow = act + (size_t)a * (size_t)inter;
    float *yrow = y + (size_t)a * (size_t)hidden;
    const int row0 = (blockIdx.y * kGemvWaves + wave) * rows_per_wave;
    // eight rows at a time (rows_per_wave is a multiple of 4; an odd group of four runs half empty)
    for (int r = 0; r < rows_per_wave; r += 8) {
        if (row0 + r >= hidden) break;
        const int live = rows_per_wave - r < 8 ? rows_per_wave - r : 8;
        const uint8_t *rowp[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int row = (j < live && row0 + r + j < hidden) ? row0 + r + j : (row0 + r < hidden ? row0 + r : hidden - 1);
            rowp[j] = de + (size_t)row * row_bytes;
        }
        float p[8];
        rows_partial_f<WT, VEC, 8>(rowp, arow, inter, lane, p);
#pragma unroll
        for (int j = 0; j < 8; j++) p[j] = wave_sum(p[j]);
        if (lane < live && row0 + r + lane < hidden) {
            float v = p[0];
#pragma unroll
            for (int j = 1; j < 8; j++) v = lane == j ? p[j] : v;
            yrow[row0 + r + lane] = v;
        }
    }
}

// ------------------------------------------------------------------------------------------
// down + combine in one launch (quantized down bank, top_k <= kDcWaves*KPW <= 16): blockIdx.x = token,
// blockIdx.y = tile of NIT*rows_per_it output rows.  The kDcWaves waves split the token's experts
// in ascending-id order, KPW each; their row sums meet in LDS and are combined in that same
// order, multiply and add rounded separately.
// ------------------------------------------------------------------------------------------
template <int WT, int UPL, int NIT, int KPW, int kDcWaves = 4, bool ORDERED = false>
__global__ __launch_bounds__(64 * kDcWaves) void down_combine_q_kernel(
    const uint8_t *down /* not __restrict__: the code fences below must order its loads */, QAct actq, const int32_t *__restrict__ ids, const float *__restrict__ weights,
    int k, int hidden, int inter, int n_experts, const float *__restrict__ residual, float *__restrict__ out,
    unsigned long long *epoch_bump) {
    constexpr int KMAX = kDcWaves * KPW;
    // the launch before this one (gate_up_fused_kernel) has finished with the epoch: move it on for the next
    if (epoch_bump != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && (!ORDERED || blockIdx.z == 0) && threadIdx.x == 0) *epoch_bump = *epoch_bump + 1ULL;
    extern __shared__ float s_mem[];  // [KMAX][rows_per_block] row sums, then [KMAX] weights
    MUMMU_PHASE(0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // grid = (token, row tile), or ORDERED: (row tile modulo 8, token, row tile / 8)
    int t = blockIdx.x, tile = blockIdx.y;
    if constexpr (ORDERED) {
        t = blockIdx.y;
        tile = blockIdx.z * kXcds + blockIdx.x;
    }
    const RowSplit rs = row_split(inter);
    const int sub = lane >> rs.group_log2, unit0 = lane & (rs.group - 1);
    const int rows_per_block = NIT * rs.rows_per_it;
    const int row0 = tile * rows_per_block;
    if (ORDERED && row0 >= hidden) return;  // (the eight columns cover a whole number of tiles or a few more)
    float *s_y = s_mem;
    float *s_w = s_mem + KMAX * rows_per_block;
    const size_t row_bytes = type_row_bytes(WT, inter);

    // rank of every slot by ascending expert id (ids of one token are distinct); lanes >= k idle
    const int my_id = lane < k ? ids[(size_t)t * k + lane] : 0x7FFFFFFF;
    const float my_w = lane < k ? weights[(size_t)t * k + lane] : 0.0f;
    int rank = 0;
#pragma unroll
    for (int j = 0; j < KMAX; j++) {
        const int o = __builtin_amdgcn_readlane(my_id, j);
        rank += (j < k) && (o < my_id || (o == my_id && j < lane));
    }
    // this wave's positions p = wave*KPW + i in the ascending order
    int e_p[KPW], a_p[KPW];
    bool on_p[KPW];
#pragma unroll
    for (int i = 0; i < KPW; i++) {
        const int p = wave * KPW + i;
        const unsigned long long m = __ballot(lane < k && rank == p);
        on_p[i] = m != 0ull;
        const int src = on_p[i] ? (int)__builtin_ctzll(m) : 0;
        e_p[i] = __builtin_amdgcn_readlane(my_id, src);
        a_p[i] = t * k + src;
        on_p[i] = on_p[i] && (unsigned)e_p[i] < (unsigned)n_experts;
        const float wp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), src));
        if (lane == 0) s_w[p] = on_p[i] ? wp : 0.0f;
    }

    MUMMU_PHASE(1);
    // same software pipeline as gate/up, over the wave's KPW*NIT (expert, row iteration) steps
    RawRow<WT, UPL> rd[KPW][NIT];
    LaneAct<UPL> la[KPW];
    auto fetch = [&](int step) {
        const int i = step / NIT, it = step % NIT;
        const uint8_t *de = down + (size_t)uniform_index(on_p[i] ? e_p[i] : 0) * (size_t)hidden * row_bytes;
        const int row = row0 + it * rs.rows_per_it + sub;
        const bool ok = on_p[i] && row < hidden;
        load_row<WT, UPL>(de, (uint32_t)(ok ? row : 0) * (uint32_t)row_bytes, unit0, rs.units, ok, rd[i][it]);
    };
    constexpr int STEPS = KPW * NIT;
    constexpr int AHEAD = STEPS < 2 ? STEPS : 2;
#pragma unroll
    for (int i = 0; i < KPW; i++) load_lane_act<WT, UPL>(actq, (size_t)(on_p[i] ? a_p[i] : 0), inter, unit0, rs.units, la[i]);
#pragma unroll
    for (int st = 0; st < AHEAD; st++) fetch(st);
    MUMMU_CODE_FENCE();
    float part[KPW * NIT];
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        if (st + AHEAD < STEPS) fetch(st + AHEAD);
        MUMMU_CODE_FENCE();
        part[st] = dot_row<WT, UPL>(rd[st / NIT][st % NIT], unit0, la[st / NIT]);
        MUMMU_CODE_FENCE();
    }
    MUMMU_PHASE(2);
    dispatch_group(rs.group, [&](auto group_tag) {
        constexpr int GROUP = decltype(group_tag)::value;
        const int offset = reduce_partials<KPW * NIT, GROUP>(part, lane);
        constexpr int count = reduced_count<KPW * NIT, GROUP>();
        constexpr int width = GROUP < 16 ? GROUP : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < count; j++) {
                const int idx = offset + j;
                const int i = idx / NIT, it = idx % NIT;
                s_y[(wave * KPW + i) * rows_per_block + it * rs.rows_per_it + sub] = part[j];
            }
        }
    });
    MUMMU_PHASE(3);
    __syncthreads();
    MUMMU_PHASE(4);
    for (int r = threadIdx.x; r < rows_per_block; r += blockDim.x) {
        const int row = row0 + r;
        if (row >= hidden) continue;
        float sum = 0.0f;
        for (int p = 0; p < k; p++) sum = __fadd_rn(sum, __fmul_rn(s_w[p], s_y[p * rows_per_block + r]));
        const size_t o = (size_t)t * (size_t)hidden + row;
        out[o] = residual ? __fadd_rn(residual[o], sum) : sum;
    }
    MUMMU_PHASE(5);
}

// ------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------
// Float rows: rows per wave so that a launch has a few thousand waves without tiny tiles.
static int pick_rows_per_wave(int out_dim, int n_assign) {
    int rpw = 1;
    while ((long)((out_dim + rpw * 2 - 1) / (rpw * 2)) * n_assign >= 4096 && rpw < 64) rpw *= 2;
    return rpw < 4 ? 4 : rpw;
}

template <int WT>
static hipError_t launch_gate_up_t(const ExpertBanks &b, const float *x, QAct xq, const int32_t *ids, int n_assign,
                                   int k, int fixed_expert, float *act, QAct actq, int32_t *flags, hipStream_t s) {
    constexpr bool quant = is_quant_type(WT);
    const bool actq_out = is_quant_type(b.down_type);
    const int slots = fixed_expert >= 0 ? 1 : k;  // n_assign = tokens * slots
    if constexpr (quant) {
        const RowSplit rs = row_split(b.hidden);
        const int upl = (rs.units + 63) / 64;
#define MUMMU_GUQ(UPL, NIT)                                                                                     \
    do {                                                                                                        \
        int waves = 4;                                                                                          \
        while (waves * (NIT)*rs.rows_per_it < 16) waves *= 2; /* whole 16-element activation blocks */          \
        const int rpb = waves * (NIT)*rs.rows_per_it;                                                           \
        const int tiles = (b.inter + rpb - 1) / rpb, tokens = n_assign / slots;                                 \
        dim3 grid(slots, tiles, tokens), block(64 * waves);                                                     \
        const bool ordered = tile_order_grid(tokens >= b.tile_order_from && fixed_expert < 0 && actq_out, tokens, slots * tokens, tiles, grid); \
        const size_t lds = sizeof(float) * (size_t)rpb;                                                         \
        if (ordered)                                                                                            \
            launch_kernel(gate_up_q_kernel<WT, UPL, NIT, true, 0, true>, grid, block, lds, s,                              \
                b.gate, b.up, xq, ids, k, fixed_expert, b.hidden, b.inter, b.n_experts, act, actq, flags, RouteInline());      \
        else if (actq_out)                                                                                      \
            launch_kernel(gate_up_q_kernel<WT, UPL, NIT, true>, grid, block, lds, s,                                       \
                b.gate, b.up, xq, ids, k, fixed_expert, b.hidden, b.inter, b.n_experts, act, actq, flags, RouteInline());      \
        else                                                                                                    \
            launch_kernel(gate_up_q_kernel<WT, UPL, NIT, false>, grid, block, lds, s,                                      \
                b.gate, b.up, xq, ids, k, fixed_expert, b.hidden, b.inter, b.n_experts, act, actq, flags, RouteInline());      \
    } while (0)
        if (upl == 1 && n_assign / slots >= 8 && fixed_expert < 0 && b.inter % 32 == 0) MUMMU_GUQ(1, 8);  // (as launch_gate_up_routed)
        else if (upl == 1) MUMMU_GUQ(1, 4);
        else if (upl == 2) MUMMU_GUQ(2, 2);
        else if (upl <= 4) MUMMU_GUQ(4, 1);
        else return hipErrorInvalidValue;
#undef MUMMU_GUQ
    } else {
        const int rpw = pick_rows_per_wave(b.inter, n_assign);
        dim3 block(64 * kGemvWaves), grid(slots, (b.inter + rpw * kGemvWaves - 1) / (rpw * kGemvWaves), n_assign / slots);
        const bool vec = b.hidden % 4 == 0 && (((uintptr_t)x & 15) == 0);
        constexpr int WIDE = WT == T_F32 ? 4 : 8;  // 16 bytes of a weight row per lane and load
        if (vec && b.hidden % WIDE == 0 && ((((uintptr_t)b.gate | (uintptr_t)b.up) & 15) == 0))
            launch_kernel(gate_up_f_kernel<WT, WIDE>, grid, block, 0, s, b.gate, b.up, x, ids, k, fixed_expert, b.hidden, b.inter,
                                                           b.n_experts, rpw, act, flags, RouteInline());
        else if (vec)
            launch_kernel(gate_up_f_kernel<WT, 4>, grid, block, 0, s, b.gate, b.up, x, ids, k, fixed_expert, b.hidden, b.inter,
                                                           b.n_experts, rpw, act, flags, RouteInline());
        else
            launch_kernel(gate_up_f_kernel<WT, 1>, grid, block, 0, s, b.gate, b.up, x, ids, k, fixed_expert, b.hidden, b.inter,
                                                           b.n_experts, rpw, act, flags, RouteInline());
        if (actq_out) {  // float gate/up feeding a quantized down bank: quantize the f32 act rows
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            return launch_quantize_rows(act, n_assign, b.inter, actq, s);
        }
    }
    return hipGetLastError();
}

hipError_t launch_gate_up(const ExpertBanks &b, const float *x, QAct xq, const int32_t *ids, int n_assign, int k,
                          int fixed_expert, float *act, QAct actq, int32_t *flags, hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    if (b.gate_type != b.up_type) return hipErrorInvalidValue;
    if (n_assign / (fixed_expert >= 0 ? 1 : k) > 65535) return hipErrorInvalidValue;
    return with_bank_type(b.gate_type, [&](auto tag) {
        return launch_gate_up_t<decltype(tag)::value>(b, x, xq, ids, n_assign, k, fixed_expert, act, actq, flags, s);
    });
}

// Float banks, few tokens: gate/up with the routing inside (one launch less), then down + combine
// in one launch.
bool float_decode_fused(const ExpertBanks &b, int k) {
    auto fl = [](int t) { return t == T_F32 || t == T_F16 || t == T_BF16; };
    return fl(b.gate_type) && b.gate_type == b.up_type && fl(b.down_type) && b.n_experts <= 512 && k >= 1 && k <= b.n_experts && k <= 16;
}

template <int WT>
static hipError_t launch_gate_up_f_routed_t(const ExpertBanks &b, const float *x, const RouteInline &route, int n_tokens, int k,
                                            float *act, int32_t *flags, hipStream_t s) {
    const int rpw = pick_rows_per_wave(b.inter, n_tokens * k);
    dim3 block(64 * kGemvWaves), grid(k, (b.inter + rpw * kGemvWaves - 1) / (rpw * kGemvWaves), n_tokens);
    constexpr int WIDE = WT == T_F32 ? 4 : 8;
    const bool vec = b.hidden % 4 == 0 && (((uintptr_t)x & 15) == 0);
    const bool wide = vec && b.hidden % WIDE == 0 && ((((uintptr_t)b.gate | (uintptr_t)b.up) & 15) == 0);
#define MUMMU_GUF(VEC, JN)                                                                                              \
    launch_kernel(gate_up_f_kernel<WT, VEC, JN>, grid, block, 0, s, b.gate, b.up, x, (const int32_t *)nullptr, k, -1, b.hidden, \
                  b.inter, b.n_experts, rpw, act, flags, route)
#define MUMMU_GUF_JN(VEC)                                                                                               \
    do {                                                                                                                \
        if (b.n_experts <= 64) MUMMU_GUF(VEC, 1);                                                                       \
        else if (b.n_experts <= 128) MUMMU_GUF(VEC, 2);                                                                 \
        else MUMMU_GUF(VEC, 8);                                                                                         \
    } while (0)
    if (wide) MUMMU_GUF_JN(WIDE);
    else if (vec) MUMMU_GUF_JN(4);
    else MUMMU_GUF_JN(1);
#undef MUMMU_GUF_JN
#undef MUMMU_GUF
    return hipGetLastError();
}

hipError_t launch_gate_up_f_routed(const ExpertBanks &b, const float *x, const RouteInline &route, int n_tokens, int k, float *act,
                                   int32_t *flags, hipStream_t s) {
    if (n_tokens <= 0) return hipSuccess;
    if (!float_decode_fused(b, k) || n_tokens > 65535) return hipErrorInvalidValue;
    return with_bank_type(b.gate_type, [&](auto tag) {
        constexpr int WT = decltype(tag)::value;
        if constexpr (!is_quant_type(WT)) return launch_gate_up_f_routed_t<WT>(b, x, route, n_tokens, k, act, flags, s);
        else return hipErrorInvalidValue;
    });
}

// down + combine, float down bank, top_k <= 16: blockIdx.x = token, blockIdx.y = tile of 8 output rows.
// Wave w takes the token's slots w, w + 8; the row sums (the same sums, bit for bit, as down_f_kernel
// makes) meet in LDS and eight lanes add them as combine_kernel does: ascending expert id, multiply
// and add rounded separately.
template <int WT, int VEC>
__global__ __launch_bounds__(512) void down_combine_f_kernel(const uint8_t *__restrict__ down, const float *__restrict__ act,
                                                             const int32_t *__restrict__ ids, const float *__restrict__ weights,
                                                             int k, int hidden, int inter, int n_experts,
                                                             const float *__restrict__ residual, float *__restrict__ out) {
    __shared__ float s_y[16][8];
    __shared__ int s_order[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x, row0 = blockIdx.y * 8;
    if (tid < k) {
        const int id = ids[(size_t)t * k + tid];
        int rank = 0;
        for (int j = 0; j < k; j++) {
            const int o = ids[(size_t)t * k + j];
            rank += (o < id) || (o == id && j < tid);
        }
        s_order[rank] = tid;
    }
    const size_t row_bytes = type_row_bytes(WT, inter);
    for (int sl = wave; sl < k; sl += 8) {
        const int a = t * k + sl;
        const int e = ids[a];
        float p[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if ((unsigned)e < (unsigned)n_experts) {  // (a bad id was flagged by gate/up)
            const uint8_t *de = down + (size_t)e * (size_t)hidden * row_bytes;
            const uint8_t *rowp[8];
#pragma unroll
            for (int j = 0; j < 8; j++) rowp[j] = de + (size_t)(row0 + j < hidden ? row0 + j : row0) * row_bytes;
            rows_partial_f<WT, VEC, 8>(rowp, act + (size_t)a * (size_t)inter, inter, lane, p);
#pragma unroll
            for (int j = 0; j < 8; j++) p[j] = wave_sum(p[j]);
        }
        if (lane < 8) {
            float v = p[0];
#pragma unroll
            for (int j = 1; j < 8; j++) v = lane == j ? p[j] : v;
            s_y[sl][lane] = v;
        }
    }
    __syncthreads();
    if (tid < 8 && row0 + tid < hidden) {
        float sum = 0.0f;
        for (int r = 0; r < k; r++) {
            const int sl = s_order[r];
            sum = __fadd_rn(sum, __fmul_rn(weights[(size_t)t * k + sl], s_y[sl][tid]));
        }
        const size_t o = (size_t)t * (size_t)hidden + row0 + tid;
        out[o] = residual ? __fadd_rn(residual[o], sum) : sum;
    }
}

hipError_t launch_down_combine_f(const ExpertBanks &b, const float *act, const int32_t *ids, const float *weights, int n, int k,
                                 const float *residual, float *out, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (!float_decode_fused(b, k) || n > 65535) return hipErrorInvalidValue;
    return with_bank_type(b.down_type, [&](auto tag) {
        constexpr int WT = decltype(tag)::value;
        if constexpr (!is_quant_type(WT)) {
            dim3 block(512), grid(n, (b.hidden + 7) / 8);
            constexpr int WIDE = WT == T_F32 ? 4 : 8;
            if (b.inter % WIDE == 0 && (((uintptr_t)b.down & 15) == 0))
                launch_kernel(down_combine_f_kernel<WT, WIDE>, grid, block, 0, s, b.down, act, ids, weights, k, b.hidden, b.inter,
                              b.n_experts, residual, out);
            else if (b.inter % 4 == 0)
                launch_kernel(down_combine_f_kernel<WT, 4>, grid, block, 0, s, b.down, act, ids, weights, k, b.hidden, b.inter,
                              b.n_experts, residual, out);
            else
                launch_kernel(down_combine_f_kernel<WT, 1>, grid, block, 0, s, b.down, act, ids, weights, k, b.hidden, b.inter,
                              b.n_experts, residual, out);
            return hipGetLastError();
        } else {
            return hipErrorInvalidValue;
        }
    });
}

bool gate_up_routes_inline(const ExpertBanks &b, int k) {
    const RowSplit rs = row_split(b.hidden);
    return is_quant_type(b.gate_type) && b.gate_type == b.up_type && is_quant_type(b.down_type) && rs.units <= 128 &&
           b.n_experts <= 512 && k >= 1 && k <= b.n_experts && k <= 16 && b.inter % 16 == 0;
}

template <int WT, int UPL, int NIT>
static hipError_t launch_gate_up_routed_t(const ExpertBanks &b, QAct xq, const RouteInline &route, int n_tokens, int k,
                                          QAct actq, int32_t *flags, hipStream_t s) {
    const RowSplit rs = row_split(b.hidden);
    int waves = 4;
    while (waves * NIT * rs.rows_per_it < 16) waves *= 2;
    const int rpb = waves * NIT * rs.rows_per_it;
    const int tiles = (b.inter + rpb - 1) / rpb;
    dim3 grid(k, tiles, n_tokens), block(64 * waves);
    const bool ordered = tile_order_grid(n_tokens >= b.tile_order_from, n_tokens, k * n_tokens, tiles, grid);
    const size_t lds = sizeof(float) * (size_t)rpb;
#define MUMMU_GUR(JN)                                                                                                    \
    do {                                                                                                                 \
        if (ordered)                                                                                                     \
            launch_kernel(gate_up_q_kernel<WT, UPL, NIT, true, JN, true>, grid, block, lds, s, b.gate, b.up, xq,         \
                          (const int32_t *)nullptr, k, -1, b.hidden, b.inter, b.n_experts, (float *)nullptr, actq, flags, route); \
        else                                                                                                             \
            launch_kernel(gate_up_q_kernel<WT, UPL, NIT, true, JN>, grid, block, lds, s, b.gate, b.up, xq,               \
                          (const int32_t *)nullptr, k, -1, b.hidden, b.inter, b.n_experts, (float *)nullptr, actq, flags, route); \
    } while (0)
    if (b.n_experts <= 64) MUMMU_GUR(1);
    else if (b.n_experts <= 128) MUMMU_GUR(2);
    else MUMMU_GUR(8);
#undef MUMMU_GUR
    return hipGetLastError();
}

hipError_t launch_gate_up_routed(const ExpertBanks &b, QAct xq, const RouteInline &route, int n_tokens, int k, QAct actq,
                                 int32_t *flags, hipStream_t s) {
    if (n_tokens <= 0) return hipSuccess;
    if (!gate_up_routes_inline(b, k) || n_tokens > 65535) return hipErrorInvalidValue;
    const bool wide = row_split(b.hidden).units > 64;
    return with_bank_type(b.gate_type, [&](auto tag) {
        constexpr int WT = decltype(tag)::value;
        if constexpr (is_quant_type(WT)) {
            // (eight row iterations per wave from eight tokens on: the same routing and activation loads serve twice the
            // rows - 29.3 against 30.0 us at 8 tokens of the OLMoE shape, but 12.7 against 11.8 at 2)
            if (!wide && n_tokens >= 8 && b.inter % 32 == 0) return launch_gate_up_routed_t<WT, 1, 8>(b, xq, route, n_tokens, k, actq, flags, s);
            return wide ? launch_gate_up_routed_t<WT, 2, 2>(b, xq, route, n_tokens, k, actq, flags, s)
                        : launch_gate_up_routed_t<WT, 1, 4>(b, xq, route, n_tokens, k, actq, flags, s);
        } else {
            return hipErrorInvalidValue;
        }
    });
}

bool gate_up_fused_supported(const ExpertBanks &b, int k, int n_tokens, const RouterExchange &rx) {
    if (!gate_up_routes_inline(b, k) || !down_combine_supported(b, k)) return false;
    if (n_tokens < 1 || n_tokens > kExchangeTokens || b.hidden % 64 != 0 || b.hidden > 512 * kWaveRowChunks) return false;
    if (rx.wtype != T_F32 && rx.wtype != T_F16 && rx.wtype != T_BF16) return false;
    if ((((uintptr_t)rx.x | (uintptr_t)rx.w | (uintptr_t)rx.gamma | (uintptr_t)rx.xnorm_out | (uintptr_t)rx.slots) & 15) != 0) return false;
    if (rx.x == nullptr || rx.w == nullptr || rx.slots == nullptr || rx.epoch == nullptr) return false;
    if (rx.xnorm_out != nullptr && rx.gamma == nullptr) return false;
    const RowSplit rs = row_split(b.hidden);
    const int rpb = 4 * 4 * rs.rows_per_it;  // four waves, NIT = 4
    const int tiles = (b.inter + rpb - 1) / rpb;
    return (k * tiles) % 8 == 0;  // a token's workgroups spread evenly over the 8 XCDs
}

template <int WT>
static hipError_t launch_gate_up_fused_t(const ExpertBanks &b, const RouterExchange &rx, const RouteInline &route, int n_tokens,
                                         int k, QAct actq, int32_t *flags, hipStream_t s) {
    constexpr int NIT = 4;   // (measured at one token against 2 / 6 / 8 row iterations per wave: 11.7 against 11.7 / 12.8 / 12.6 us)
    const RowSplit rs = row_split(b.hidden);
    const int rpb = 4 * NIT * rs.rows_per_it;
    dim3 grid(k, (b.inter + rpb - 1) / rpb, n_tokens), block(256);
    const size_t lds = sizeof(float) * (size_t)rpb + 2 * (size_t)b.hidden + 8 * (size_t)(b.hidden / 16);
#define MUMMU_GUX(JN, EARLY) \
    launch_kernel(gate_up_fused_kernel<WT, NIT, JN, EARLY>, grid, block, lds, s, b.gate, b.up, k, b.hidden, b.inter, b.n_experts, actq, flags, route, rx)
    if (b.n_experts <= 64 && k == 8 && b.early_ids) MUMMU_GUX(1, true);
    else if (b.n_experts <= 64) MUMMU_GUX(1, false);
    else if (b.n_experts <= 128 && k == 8 && b.early_ids) MUMMU_GUX(2, true);
    else if (b.n_experts <= 128) MUMMU_GUX(2, false);
    else MUMMU_GUX(8, false);
#undef MUMMU_GUX
    return hipGetLastError();
}

hipError_t launch_gate_up_fused(const ExpertBanks &b, const RouterExchange &rx, const RouteInline &route, int n_tokens, int k,
                                QAct actq, int32_t *flags, hipStream_t s) {
    if (n_tokens <= 0) return hipSuccess;
    if (!gate_up_fused_supported(b, k, n_tokens, rx)) return hipErrorInvalidValue;
    return with_bank_type(b.gate_type, [&](auto tag) {
        constexpr int WT = decltype(tag)::value;
        if constexpr (is_quant_type(WT)) return launch_gate_up_fused_t<WT>(b, rx, route, n_tokens, k, actq, flags, s);
        else return hipErrorInvalidValue;
    });
}

template <int WT>
static hipError_t launch_down_t(const ExpertBanks &b, const float *act, QAct actq, const int32_t *ids, int n_assign,
                                int k, int fixed_expert, float *y, hipStream_t s) {
    constexpr bool quant = is_quant_type(WT);
    const int slots = fixed_expert >= 0 ? 1 : k;  // n_assign = tokens * slots
    dim3 block(64 * kGemvWaves);
    if constexpr (quant) {
        const RowSplit rs = row_split(b.inter);
        const int upl = (rs.units + 63) / 64;
#define MUMMU_DNQ(UPL, NIT)                                                                                    \
    do {                                                                                                       \
        const int rpb = kGemvWaves * (NIT)*rs.rows_per_it;                                                     \
        dim3 grid(slots, (b.hidden + rpb - 1) / rpb, n_assign / slots);                                        \
        launch_kernel(down_q_kernel<WT, UPL, NIT>, grid, block, 0, s, b.down, actq, ids, fixed_expert, b.hidden, b.inter, \
                                                           b.n_experts, y);                                    \
    } while (0)
        if (upl == 1) MUMMU_DNQ(1, 4);
        else if (upl == 2) MUMMU_DNQ(2, 2);
        else if (upl <= 4) MUMMU_DNQ(4, 1);
        else return hipErrorInvalidValue;
#undef MUMMU_DNQ
    } else {
        const int rpw = pick_rows_per_wave(b.hidden, n_assign);
        dim3 grid(slots, (b.hidden + rpw * kGemvWaves - 1) / (rpw * kGemvWaves), n_assign / slots);
        constexpr int WIDE = WT == T_F32 ? 4 : 8;
        if (b.inter % WIDE == 0 && (((uintptr_t)b.down & 15) == 0))
            launch_kernel(down_f_kernel<WT, WIDE>, grid, block, 0, s, b.down, act, ids, fixed_expert, b.hidden, b.inter, b.n_experts, rpw, y);
        else if (b.inter % 4 == 0)
            launch_kernel(down_f_kernel<WT, 4>, grid, block, 0, s, b.down, act, ids, fixed_expert, b.hidden, b.inter, b.n_experts, rpw, y);
        else
            launch_kernel(down_f_kernel<WT, 1>, grid, block, 0, s, b.down, act, ids, fixed_expert, b.hidden, b.inter, b.n_experts, rpw, y);
    }
    return hipGetLastError();
}

hipError_t launch_down(const ExpertBanks &b, const float *act, QAct actq, const int32_t *ids, int n_assign, int k,
                       int fixed_expert, float *y, hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    if (n_assign / (fixed_expert >= 0 ? 1 : k) > 65535) return hipErrorInvalidValue;
    return with_bank_type(b.down_type, [&](auto tag) {
        return launch_down_t<decltype(tag)::value>(b, act, actq, ids, n_assign, k, fixed_expert, y, s);
    });
}

bool down_combine_supported(const ExpertBanks &b, int k) {
    return is_quant_type(b.down_type) && k <= 16 && (row_split(b.inter).units + 63) / 64 <= 2;
}

template <int WT>
static hipError_t launch_down_combine_t(const ExpertBanks &b, QAct actq, const int32_t *ids, const float *weights, int n,
                                        int k, const float *residual, float *out, hipStream_t s, unsigned long long *epoch_bump) {
    const RowSplit rs = row_split(b.inter);
    const int upl = (rs.units + 63) / 64;
#define MUMMU_DC(UPL, NIT, KPW, WAVES)                                                                             \
    do {                                                                                                           \
        const int rpb = (NIT)*rs.rows_per_it;                                                                      \
        const int tiles = (b.hidden + rpb - 1) / rpb;                                                              \
        dim3 grid(n, tiles), block(64 * (WAVES));                                                                  \
        const bool ordered = tile_order_grid(n >= b.tile_order_from, n, n, tiles, grid);                                    \
        const size_t lds = sizeof(float) * (size_t)((WAVES) * (KPW)) * (size_t)(rpb + 1);                          \
        if (ordered)                                                                                               \
            launch_kernel(down_combine_q_kernel<WT, UPL, NIT, KPW, WAVES, true>, grid, block, lds, s, b.down, actq, ids, weights, k, \
                          b.hidden, b.inter, b.n_experts, residual, out, epoch_bump);                              \
        else                                                                                                       \
            launch_kernel(down_combine_q_kernel<WT, UPL, NIT, KPW, WAVES>, grid, block, lds, s, b.down, actq, ids, weights, k, \
                          b.hidden, b.inter, b.n_experts, residual, out, epoch_bump);                              \
    } while (0)
    // one expert per wave up to top_k 8 (eight waves, four row iterations each: measured against two experts per wave
    // in four waves and against one / two / six / eight iterations, 5.4 against 5.8 us at one token and 18.0
    // against 23.0 us at eight), two per wave beyond
    if (upl == 1) {
        if (k <= 4) MUMMU_DC(1, 4, 1, 4);
        else if (k <= 8 && n >= 3) MUMMU_DC(1, 8, 1, 8);  // (several tokens: 9.5 against 11.0 us at 4 tokens, 16.2 against 17.9 at 8; 6.1 against 5.4 at one)
        else if (k <= 8) MUMMU_DC(1, 4, 1, 8);
        else if (k <= 10) MUMMU_DC(1, 2, 2, 5);  // (ten waves of one expert: 8.7 against 7.7 us at one token, top-10 of 512)
        else if (k <= 12) MUMMU_DC(1, 2, 2, 6);
        else MUMMU_DC(1, 2, 2, 8);
    } else {
        if (k <= 4) MUMMU_DC(2, 2, 1, 4);
        else if (k <= 8) MUMMU_DC(2, 2, 2, 4);
        else MUMMU_DC(2, 2, 2, 8);
    }
#undef MUMMU_DC
    return hipGetLastError();
}

hipError_t launch_down_combine(const ExpertBanks &b, QAct actq, const int32_t *ids, const float *weights, int n, int k,
                               const float *residual, float *out, hipStream_t s, unsigned long long *epoch_bump) {
    if (n <= 0) return hipSuccess;
    if (!down_combine_supported(b, k)) return hipErrorInvalidValue;
    return with_bank_type(b.down_type, [&](auto tag) {
        constexpr int WT = decltype(tag)::value;
        if constexpr (is_quant_type(WT)) return launch_down_combine_t<WT>(b, actq, ids, weights, n, k, residual, out, s, epoch_bump);
        else return hipErrorInvalidValue;
    });
}

// ------------------------------------------------------------------------------------------
// combine: out[t] = (residual[t] +) sum over the token's slots in ascending expert id of
// w * y, multiply and add rounded separately.
// ------------------------------------------------------------------------------------------
constexpr int kCombineMaxK = 512;

// VEC4: hidden % 4 == 0, a thread takes four neighbouring columns (one 16-byte load per slot).
template <bool VEC4>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y, const int32_t *__restrict__ ids,
                                                      const float *__restrict__ weights,
                                                      const int32_t *__restrict__ inv, int k, int hidden,
                                                      const float *__restrict__ residual, float *__restrict__ out,
                                                      unsigned long long *epoch_bump) {
    // the launch before this one (decode_layer_kernel) has finished with the epoch: move it on for the next
    if (epoch_bump != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *epoch_bump = *epoch_bump + 1ULL;
    __shared__ int s_order[kCombineMaxK];
    __shared__ int s_row[kCombineMaxK];
    __shared__ float s_w[kCombineMaxK];
    const int t = blockIdx.x;
    for (int s = threadIdx.x; s < k; s += blockDim.x) {
        const int id = ids[(size_t)t * k + s];
        int rank = 0;
        for (int j = 0; j < k; j++) {
            const int o = ids[(size_t)t * k + j];
            rank += (o < id) || (o == id && j < s);
        }
        s_order[rank] = s;
    }
    __syncthreads();
    for (int s = threadIdx.x; s < k; s += blockDim.x) {
        const int a = t * k + s_order[s];
        s_w[s] = weights[a];
        s_row[s] = inv ? inv[a] : a;
    }
    __syncthreads();
    if constexpr (VEC4) {
        for (int c = 4 * (blockIdx.y * blockDim.x + threadIdx.x); c < hidden; c += 4 * gridDim.y * blockDim.x) {
            float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            for (int r = 0; r < k; r++) {
                const float4 v = *(const float4 *)(y + (size_t)s_row[r] * (size_t)hidden + c);
                const float w = s_w[r];
                sum.x = __fadd_rn(sum.x, __fmul_rn(w, v.x));
                sum.y = __fadd_rn(sum.y, __fmul_rn(w, v.y));
                sum.z = __fadd_rn(sum.z, __fmul_rn(w, v.z));
                sum.w = __fadd_rn(sum.w, __fmul_rn(w, v.w));
            }
            if (residual) {
                const float4 q = *(const float4 *)(residual + (size_t)t * hidden + c);
                sum.x = __fadd_rn(q.x, sum.x);
                sum.y = __fadd_rn(q.y, sum.y);
                sum.z = __fadd_rn(q.z, sum.z);
                sum.w = __fadd_rn(q.w, sum.w);
            }
            *(float4 *)(out + (size_t)t * hidden + c) = sum;
        }
    } else {
        for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < hidden; c += gridDim.y * blockDim.x) {
            float sum = 0.0f;
            for (int r = 0; r < k; r++) {
                const float v = y[(size_t)s_row[r] * (size_t)hidden + c];
                sum = __fadd_rn(sum, __fmul_rn(s_w[r], v));
            }
            out[(size_t)t * hidden + c] = residual ? __fadd_rn(residual[(size_t)t * hidden + c], sum) : sum;
        }
    }
}

hipError_t launch_combine(const float *y, const int32_t *ids, const float *weights, const int32_t *inv, int n, int k,
                          int hidden, const float *residual, float *out, hipStream_t s, unsigned long long *epoch_bump) {
    if (n <= 0) return hipSuccess;
    if (k > kCombineMaxK) return hipErrorInvalidValue;
    // a token's row is split over enough workgroups to have about four on every CU
    const bool vec4 = hidden % 4 == 0 && (((uintptr_t)y | (uintptr_t)out | (uintptr_t)residual) & 15) == 0;
    const int per_wg = vec4 ? 1024 : 256;   // columns a workgroup covers per pass
    int ysplit = (1024 + n - 1) / n;
    ysplit = std::max(1, std::min(ysplit, (hidden + per_wg - 1) / per_wg));
    dim3 block(256), grid(n, ysplit);
    if (vec4) launch_kernel(combine_kernel<true>, grid, block, 0, s, y, ids, weights, inv, k, hidden, residual, out, epoch_bump);
    else launch_kernel(combine_kernel<false>, grid, block, 0, s, y, ids, weights, inv, k, hidden, residual, out, epoch_bump);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// shared expert: out = [residual +] (out + y * sigmoid(<gate_vec, x>)), each operation rounded on its
// own (models/qwen4exp/model.rs:786-804).  gate_vec null: the shared expert is not gated.  Every wave
// computes the token's gate logit for itself, in the router's order (eight partials per lane over
// 512-element chunks, the fixed fold, the wave sum): no launch of its own for one dot product.
// ------------------------------------------------------------------------------------------
template <int WT, bool VEC>
__device__ inline float gate_logit(const float *__restrict__ xrow, const void *__restrict__ gv, int hidden, int lane) {
    float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 4
    for (int base = lane * 8; base < hidden; base += 512) {
        if constexpr (VEC) {  // hidden % 8 == 0, both rows 16-byte aligned: the lane's 8 elements are inside the row
            const float4 p = *(const float4 *)(xrow + base), q = *(const float4 *)(xrow + base + 4);
            const float xv[8] = {p.x, p.y, p.z, p.w, q.x, q.y, q.z, q.w};
            float w[8];
            if constexpr (WT == T_F32) {
                const float4 u = *(const float4 *)((const float *)gv + base), v = *(const float4 *)((const float *)gv + base + 4);
                w[0] = u.x; w[1] = u.y; w[2] = u.z; w[3] = u.w; w[4] = v.x; w[5] = v.y; w[6] = v.z; w[7] = v.w;
            } else {
                const uint4 u = *(const uint4 *)((const uint16_t *)gv + base);
                const uint32_t r[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const uint16_t hb = (uint16_t)((r[j / 2] >> (16 * (j & 1))) & 0xFFFFu);
                    w[j] = WT == T_F16 ? half_bits_to_float(hb) : bf16_bits_to_float(hb);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; j++) a[j] = __builtin_fmaf(xv[j], w[j], a[j]);
            continue;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = base + j;
            float w = 0.0f, xv = 0.0f;  // +0 leaves a partial unchanged
            if (i < hidden) {
                xv = xrow[i];
                if constexpr (WT == T_F32) w = ((const float *)gv)[i];
                else if constexpr (WT == T_F16) w = half_bits_to_float(((const uint16_t *)gv)[i]);
                else w = bf16_bits_to_float(((const uint16_t *)gv)[i]);
            }
            a[j] = __builtin_fmaf(xv, w, a[j]);
        }
    }
    const float sum = __fadd_rn(__fadd_rn(__fadd_rn(a[0], a[4]), __fadd_rn(a[1], a[5])),
                                __fadd_rn(__fadd_rn(a[2], a[6]), __fadd_rn(a[3], a[7])));
    return wave_sum(sum);
}

template <int WT, bool VEC>
__global__ __launch_bounds__(256) void shared_add_kernel(float *__restrict__ out, const float *__restrict__ y,
                                                         const float *__restrict__ x, const void *__restrict__ gate_vec,
                                                         const float *__restrict__ residual, int hidden) {
    const int t = blockIdx.x;
    float g = 1.0f;
    if (gate_vec) {
        const float logit = gate_logit<WT, VEC>(x + (size_t)t * (size_t)hidden, gate_vec, hidden, threadIdx.x & 63);
        g = __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-logit)));
    }
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < hidden; c += gridDim.y * blockDim.x) {
        const size_t o = (size_t)t * (size_t)hidden + c;
        const float shared = gate_vec ? __fmul_rn(y[o], g) : y[o];
        const float v = __fadd_rn(out[o], shared);
        out[o] = residual ? __fadd_rn(residual[o], v) : v;
    }
}

hipError_t launch_shared_add(float *out, const float *y, const float *x, const void *gate_vec, int gate_vec_type,
                             const float *residual, int n, int hidden, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    int ysplit = n >= 64 ? 1 : (hidden + 255) / 256;
    dim3 grid(n, ysplit), block(256);
    const bool vec = hidden % 8 == 0 && ((((uintptr_t)x | (uintptr_t)gate_vec) & 15) == 0);
#define MUMMU_SA(WT)                                                                                              \
    do {                                                                                                          \
        if (vec) launch_kernel(shared_add_kernel<WT, true>, grid, block, 0, s, out, y, x, gate_vec, residual, hidden); \
        else launch_kernel(shared_add_kernel<WT, false>, grid, block, 0, s, out, y, x, gate_vec, residual, hidden);    \
    } while (0)
    switch (gate_vec ? gate_vec_type : T_F32) {
    case T_F32: MUMMU_SA(T_F32); break;
    case T_F16: MUMMU_SA(T_F16); break;
    case T_BF16: MUMMU_SA(T_BF16); break;
    default: return hipErrorInvalidValue;
    }
#undef MUMMU_SA
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// gate energy (nn/moe.rs:508-521): energy[t] = sum over the intermediate width of
// silu(<gate_i, x_t>)^2, the gate product only.  w holds the expert's gate rows as f32 (the
// dequantizer's output or an F32 bank).  A workgroup takes kEnergyRows token rows (in LDS) and
// kEnergyGate gate rows (four per wave, a wave-wide dot each); the squares of a tile are added in
// a fixed order (per wave by row, then the four waves pairwise), the tiles by the second kernel in
// ascending order.  Not a hot path: the reference calls it only to pick rows in its skip mode.
// ------------------------------------------------------------------------------------------
constexpr int kEnergyRows = 4, kEnergyGate = 16;

__global__ __launch_bounds__(256) void gate_energy_partial_kernel(const float *__restrict__ w, const float *__restrict__ x,
                                                                  int rows, int hidden, int inter,
                                                                  float *__restrict__ partial) {
    extern __shared__ float s_x[];  // kEnergyRows * hidden
    __shared__ float s_e[4][kEnergyRows];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r0 = blockIdx.x * kEnergyRows, tile = blockIdx.y;
    for (int idx = tid; idx < kEnergyRows * hidden; idx += 256) {
        const int r = idx / hidden, c = idx - r * hidden;
        s_x[idx] = r0 + r < rows ? x[(size_t)(r0 + r) * (size_t)hidden + c] : 0.0f;
    }
    __syncthreads();
    float e[kEnergyRows];
#pragma unroll
    for (int r = 0; r < kEnergyRows; r++) e[r] = 0.0f;
    for (int j = 0; j < kEnergyGate / 4; j++) {
        const int i = tile * kEnergyGate + 4 * j + wave;  // uniform over the wave
        if (i >= inter) break;
        const float *wr = w + (size_t)i * (size_t)hidden;
        float acc[kEnergyRows];
#pragma unroll
        for (int r = 0; r < kEnergyRows; r++) acc[r] = 0.0f;
        for (int c = lane; c < hidden; c += 64) {
            const float wv = wr[c];
#pragma unroll
            for (int r = 0; r < kEnergyRows; r++) acc[r] = fmaf(wv, s_x[r * hidden + c], acc[r]);
        }
#pragma unroll
        for (int r = 0; r < kEnergyRows; r++) {
            const float sl = det_silu(wave_sum(acc[r]));
            e[r] = __fadd_rn(e[r], __fmul_rn(sl, sl));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < kEnergyRows; r++) s_e[wave][r] = e[r];
    }
    __syncthreads();
    if (tid < kEnergyRows && r0 + tid < rows)
        partial[(size_t)tile * (size_t)rows + (size_t)(r0 + tid)] =
            __fadd_rn(__fadd_rn(s_e[0][tid], s_e[1][tid]), __fadd_rn(s_e[2][tid], s_e[3][tid]));
}

__global__ __launch_bounds__(256) void gate_energy_sum_kernel(const float *__restrict__ partial, int tiles, int rows,
                                                              float *__restrict__ energy) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    float e = 0.0f;
    for (int t = 0; t < tiles; t++) e = __fadd_rn(e, partial[(size_t)t * (size_t)rows + r]);
    energy[r] = e;
}

int gate_energy_tiles(int inter) { return (inter + kEnergyGate - 1) / kEnergyGate; }

hipError_t launch_gate_energy(const float *w, const float *x, int rows, int hidden, int inter, float *partial, float *energy,
                              hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    const size_t lds = sizeof(float) * (size_t)kEnergyRows * (size_t)hidden;
    if (lds > 128 * 1024 || hidden < 1 || inter < 1) return hipErrorInvalidValue;
    const int tiles = gate_energy_tiles(inter);
    if (tiles > 65535) return hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)gate_energy_partial_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    launch_kernel(gate_energy_partial_kernel, dim3((rows + kEnergyRows - 1) / kEnergyRows, tiles), dim3(256), lds, s, w, x, rows,
                  hidden, inter, partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    launch_kernel(gate_energy_sum_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, (const float *)partial, tiles, rows, energy);
    return hipGetLastError();
}

}  // namespace mummu
