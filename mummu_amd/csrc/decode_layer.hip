// Decode step of one MoE layer on block-quantized banks in ONE expert launch: router logits, routing, gate/up,
// SwiGLU and the down product of every routed expert (nn/moe.rs:296-328 and models/qwen4exp/experts.rs:1092-1150,
// per routed (token, expert) pair: down(silu(gate.x) * (up.x))).  The weighted sum over a token's experts, in
// ascending expert id with two roundings (nn/moe.rs:1590-1601), is left to combine_kernel.
//
// top_k = 8 and the grid (slot, row tile, token): workgroups are dealt to the chip's 8 XCDs round-robin by linear id,
// so all workgroups of one expert slot run on ONE XCD and share its L2.  After the prologue (decode_route_prologue)
// a workgroup computes its tile of gate/up rows, quantizes silu(gate) * up to 16-bit blocks and publishes them as
// tagged 16-byte pieces in a table of its XCD - a plain store that stays in that L2.  It then collects the other
// blocks of its slot's hidden row from the same table with device-scope loads and multiplies its share of the
// expert's down rows, whose bytes it asked for while the gate/up rows were still streaming: the down product costs
// one exchange inside an L2 instead of a launch, and its weight stream hides behind the wait for the slowest
// workgroup.  Nothing crosses XCDs inside the launch: every slot leaves its own row of down sums in y.
//
// EARLY: the workgroups do not wait for the routing.  Wave 0 stops at the eight largest LOGITS,
// the workgroup starts its rows on the expert of its slot's rank, and wave 0 confirms the pick behind its first row
// loads - the softmax, then a check that rounds on the probabilities would choose the same experts in the same order
// (route_token_checked8), with the rounds themselves only where the check fails.  A slot whose expert the routing then
// names differently (probabilities that tie or cross where the logits do not: the tie goes to the lower id) does its
// rows again for that expert, in every workgroup of the slot alike.  Same bits as routing first.
//
// Every wait is bounded (spin_ticks of the 100 MHz clock).  A workgroup that does not find a block - workgroups
// placed otherwise than assumed, not all resident at once, or a tiny bound set by a test - computes that block's
// gate/up rows itself with the same code: the same bits, only slower.
#include "device_utils.h"
#include "kernels.h"
#include "gemv_common.h"
#include "route_common.h"
#include "decode_parts.h"

#include <cstdint>
#include <type_traits>

MUMMU_TRACE_UNIT(decode_layer)

namespace mummu {

// One 16-element block of a hidden row as it travels through the table: four 16-byte pieces of three data words
// and a tag.  hi / lo: the block's 16 high / low bytes as four words each.
//   piece 0 = {hi0, hi1, hi2}   piece 1 = {hi3, lo0, lo1}   piece 2 = {lo2, lo3, scale}   piece 3 = {sum, 0, 0}
__device__ __forceinline__ u32x4 act_piece_from_lds(const int8_t *s_hi, const int8_t *s_lo, const float *s_scale, const int *s_sum,
                                                    int blk, int piece, unsigned tag) {
    const uint32_t *h = (const uint32_t *)(s_hi + 16 * blk), *l = (const uint32_t *)(s_lo + 16 * blk);
    u32x4 r;
    r.x = piece == 0 ? h[0] : (piece == 1 ? h[3] : (piece == 2 ? l[2] : (uint32_t)s_sum[blk]));
    r.y = piece == 0 ? h[1] : (piece == 1 ? l[0] : (piece == 2 ? l[3] : 0u));
    r.z = piece == 0 ? h[2] : (piece == 1 ? l[1] : (piece == 2 ? __float_as_uint(s_scale[blk]) : 0u));
    r.w = tag;
    return r;
}

__device__ __forceinline__ void act_piece_to_lds(const u32x4 &r, int8_t *s_hi, int8_t *s_lo, float *s_scale, int *s_sum, int blk,
                                                 int piece) {
    uint32_t *h = (uint32_t *)(s_hi + 16 * blk), *l = (uint32_t *)(s_lo + 16 * blk);
    if (piece == 0) {
        h[0] = r.x; h[1] = r.y; h[2] = r.z;
    } else if (piece == 1) {
        h[3] = r.x; l[0] = r.y; l[1] = r.z;
    } else if (piece == 2) {
        l[2] = r.x; l[3] = r.y; s_scale[blk] = __uint_as_float(r.z);
    } else {
        s_sum[blk] = (int)r.x;
    }
}

// The rows s_act[0 .. rows_per_block) of tile `tile` of a hidden row -> 16-bit blocks in the workgroup's LDS copy
// of that row (the arithmetic of quantize16: what the other decode kernels store to global memory).
__device__ __forceinline__ void quantize_tile_to_lds(const float *s_act, int rows_per_block, int tile, int inter, int8_t *s_hi,
                                                     int8_t *s_lo, float *s_scale, int *s_sum) {
    if ((int)threadIdx.x < rows_per_block) {  // whole 16-lane rows: rows_per_block is a multiple of 16
        const int row = tile * rows_per_block + (int)threadIdx.x;
        const bool on = row < inter;  // inter % 16 == 0: a 16-lane row is all on or all off
        int hi, lo, sum;
        float scale;
        quantize16(on ? s_act[threadIdx.x] : 0.0f, hi, lo, scale, sum);
        if (on) {
            s_hi[row] = (int8_t)hi;
            s_lo[row] = (int8_t)lo;
            if ((row & 15) == 0) {
                s_scale[row >> 4] = scale;
                s_sum[row >> 4] = sum;
            }
        }
    }
}

constexpr int kDlWaves = 4;  // waves per workgroup (eight, in half as many workgroups, measured the same: 14.9 us per layer)

template <int WT, int DT, int NITD, int RJN, bool EARLY>
// (the three banks are not __restrict__: the code fences between the row loads must order them - gate/up rows first,
// the down rows behind them - and the compiler moves loads of restrict pointers across such a fence as it likes)
__global__ __launch_bounds__(64 * kDlWaves) void decode_layer_kernel(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                                                           int k, int hidden, int inter, int n_experts, int32_t *__restrict__ flags,
                                                           RouteInline route, RouterExchange rx, LayerExchange lx, PendingSum ps) {
    constexpr int NIT = 4;
    extern __shared__ float s_dyn[];  // gate/up results of a tile | the token's 16-bit row | the slot's 16-bit hidden row
    __shared__ __attribute__((aligned(16))) DecodeShared<RJN> sh;
    __shared__ unsigned long long s_missing[4];   // (256 pieces at most: the first four waves look for them)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.z, slot = blockIdx.x, tile = blockIdx.y;  // grid = (slot, row tile, token)
    const int a = t * gridDim.x + slot;
    const RowSplit rs = row_split(hidden);
    const int unit0 = lane & (rs.group - 1);
    const int rows_per_block = NIT * rs.rows_per_it * kDlWaves;
    float *s_act = s_dyn;
    int8_t *s_xhi = (int8_t *)(s_dyn + rows_per_block);
    int8_t *s_xlo = s_xhi + hidden;
    float *s_xscale = (float *)(s_xlo + hidden);
    int *s_xsum = (int *)(s_xscale + hidden / 16);
    int8_t *s_ahi = (int8_t *)(s_xsum + hidden / 16);
    int8_t *s_alo = s_ahi + inter;
    float *s_ascale = (float *)(s_alo + inter);
    int *s_asum = (int *)(s_ascale + inter / 16);
    MUMMU_PHASE(0);
    // while wave 0 routes, wave 1 of every workgroup adds up the rows an earlier launch left to this one
    auto side_work = [&]() {
        if (ps.n > 0 && wave == 1)
            pending_sum_wave(ps, hidden, (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x, gridDim.x * gridDim.y * gridDim.z);
    };
    RouteCarry<RJN> carry;
    const unsigned long long epoch = decode_route_prologue<RJN, decltype(side_work), EARLY>(k, hidden, n_experts, flags, route, rx, sh, s_xhi, s_xlo,
                                                                                            s_xscale, s_xsum, side_work, &carry);
    LaneAct<1> la;
    load_lane_act_lds<WT>(s_xhi, s_xlo, s_xscale, s_xsum, unit0, rs.units, la);
    // EARLY: the slot's expert by the rank of its logit, the routing proper still to come (route_rest, below)
    int e = EARLY ? sh.early_ids[slot] : sh.ids[slot];
    if ((unsigned)e >= (unsigned)n_experts) {  // (the same for every workgroup of the slot: nobody waits for this one)
        if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
        return;
    }

    // this wave's share of the expert's down rows: NITD iterations of rows_per_it rows, asked for once every gate/up
    // row has been, so that they queue up behind them
    const RowSplit rsd = row_split(inter);
    const int subd = lane >> rsd.group_log2, unit0d = lane & (rsd.group - 1);
    const int down_rows_wg = kDlWaves * NITD * rsd.rows_per_it;
    const int drow0 = tile * down_rows_wg + wave * NITD * rsd.rows_per_it;
    const uint32_t drow_bytes = (uint32_t)type_row_bytes(DT, inter);
    const uint8_t *de = down + (size_t)uniform_index(e) * (size_t)hidden * drow_bytes;
    RawRow<DT, 1> rd[NITD];
    auto fetch_down = [&](float after) {
        // (an offset of zero that the compiler cannot see through: the loads below wait for the value it is made of)
        unsigned zero;
        asm volatile("v_and_b32 %0, 0, %1" : "=v"(zero) : "v"(after));
#pragma unroll
        for (int i = 0; i < NITD; i++) {
            const int row = drow0 + i * rsd.rows_per_it + subd;
            const bool ok = row < hidden;
            load_row<DT, 1>(de, (uint32_t)(ok ? row : 0) * drow_bytes + zero, unit0d, rsd.units, ok, rd[i]);
        }
    };
    // (asked for behind the dots of iteration 0 / 1 / 2 / 3, one token on the OLMoE shape: 15.5 / 14.8 / 14.9 / 15.3 us per layer;
    // together with the gate/up rows, which is where the compiler puts every load it is free to move: 15.0)
    if constexpr (EARLY) {
        // wave 0 routes while the first rows of its share are on their way
        auto route_rest = [&]() {
            if (wave == 0) decode_route_finish<RJN, true>(carry.l, k, n_experts, flags, route, rx, sh);
        };
        gate_up_tile<WT, 1, NIT, true, false, decltype(fetch_down), 1, decltype(route_rest)>(gate, up, e, a, la, rs, hidden, inter, nullptr, QAct(),
                                                                                             s_act, tile, fetch_down, route_rest);
        __syncthreads();
        if (sh.ids[slot] != e) {
            // the routing gives this slot another expert than its logit's rank did (the same finding in every workgroup of
            // the slot): the rows again, for that one
            e = sh.ids[slot];
            if ((unsigned)e >= (unsigned)n_experts) {
                if (threadIdx.x == 0) atomicAdd(&flags[FLAG_BAD_ID], 1);
                return;
            }
            de = down + (size_t)uniform_index(e) * (size_t)hidden * drow_bytes;
            gate_up_tile<WT, 1, NIT, true, false, decltype(fetch_down), 1>(gate, up, e, a, la, rs, hidden, inter, nullptr, QAct(), s_act, tile, fetch_down);
            __syncthreads();
        }
    } else {
        gate_up_tile<WT, 1, NIT, true, false, decltype(fetch_down), 1>(gate, up, e, a, la, rs, hidden, inter, nullptr, QAct(), s_act, tile, fetch_down);
        __syncthreads();
    }
    MUMMU_PHASE(4);

    // this tile's blocks: into the LDS copy of the slot's hidden row, and out to the XCD's table
    const int blocks_per_tile = rows_per_block >> 4, n_blocks = inter >> 4;
    quantize_tile_to_lds(s_act, rows_per_block, tile, inter, s_ahi, s_alo, s_ascale, s_asum);
    __syncthreads();
    u32x4 *table = (u32x4 *)lx.act_slots +
                   ((((size_t)xcc_id() * kExchangeTokens + (size_t)t) * 8 + (size_t)slot) * (size_t)kActBlocksMax) * 4;
    const unsigned pos0 = (unsigned)((t * 8 + slot) * kActBlocksMax) * 4u;
    if ((int)threadIdx.x < 4 * blocks_per_tile) {
        const int blk = tile * blocks_per_tile + ((int)threadIdx.x >> 2), piece = (int)threadIdx.x & 3;
        if (blk < n_blocks)
            table[blk * 4 + piece] =
                act_piece_from_lds(s_ahi, s_alo, s_ascale, s_asum, blk, piece, act_piece_tag(epoch, rx.salt, pos0 + (unsigned)(blk * 4 + piece)));
    }
    MUMMU_PHASE(14);
    // (the rows this launch is still waiting for have all been asked for: the next launch's router is read ahead behind them)
    warm_next(lx.warm, lx.warm_bytes);

    // the other blocks of the row: thread i looks for piece i & 3 of block i >> 2
    {
        const int blk = (int)threadIdx.x >> 2, piece = (int)threadIdx.x & 3;
        const bool own = blk >= tile * blocks_per_tile && blk < (tile + 1) * blocks_per_tile;
        bool have = blk >= n_blocks || own;   // (threads from 256 on: blk >= kActBlocksMax >= n_blocks)
        const unsigned want = act_piece_tag(epoch, rx.salt, pos0 + threadIdx.x);
        const unsigned long long t_begin = wall_clock64();
        bool complete = __all(have);
        while (!complete && rx.spin_ticks != 0u) {  // (a bound of 0: do not look at the table at all)
            if (!have) {
                const u32x4 r = load_device_scope_b128(table + threadIdx.x);
                if (r.w == want) {
                    act_piece_to_lds(r, s_ahi, s_alo, s_ascale, s_asum, blk, piece);
                    have = true;
                }
            }
            if (__all(have)) {
                complete = true;
                break;
            }
            if (wall_clock64() - t_begin >= (unsigned long long)rx.spin_ticks) break;
            __builtin_amdgcn_s_sleep(1);
        }
        const unsigned long long missing = __ballot(!have);
        if (lane == 0 && wave < 4) s_missing[wave] = missing;
    }
    __syncthreads();
    MUMMU_PHASE(15);
    if ((s_missing[0] | s_missing[1] | s_missing[2] | s_missing[3]) != 0ull) {
        // blocks that never came: their tiles' gate/up rows are computed here (the same function of the same rows)
        if (threadIdx.x == 0 && lx.fallbacks != nullptr) atomicAdd(lx.fallbacks, 1ULL);
        const int n_tiles = (n_blocks + blocks_per_tile - 1) / blocks_per_tile;
        for (int tb = 0; tb < n_tiles; tb++) {
            const int first = tb * blocks_per_tile * 4;  // the tile's pieces: 4 * blocks_per_tile <= 32 of one wave's 64
            const unsigned long long bits = ((1ull << (4 * blocks_per_tile)) - 1ull) << (first & 63);
            if ((s_missing[first >> 6] & bits) == 0ull) continue;  // (uniform over the workgroup)
            gate_up_tile<WT, 1, NIT, true, false>(gate, up, e, a, la, rs, hidden, inter, nullptr, QAct(), s_act, tb);
            __syncthreads();
            quantize_tile_to_lds(s_act, rows_per_block, tb, inter, s_ahi, s_alo, s_ascale, s_asum);
            __syncthreads();
        }
    }

    // down rows x the slot's hidden row
    LaneAct<1> lad;
    load_lane_act_lds<DT>(s_ahi, s_alo, s_ascale, s_asum, unit0d, rsd.units, lad);
    float part[NITD];
#pragma unroll
    for (int i = 0; i < NITD; i++) part[i] = dot_row<DT, 1>(rd[i], unit0d, lad);
    MUMMU_PHASE(6);
    float *yrow = lx.y + (size_t)a * (size_t)hidden;
    dispatch_group(rsd.group, [&](auto group_tag) {
        constexpr int GROUP = decltype(group_tag)::value;
        const int offset = reduce_partials<NITD, GROUP>(part, lane);
        constexpr int count = reduced_count<NITD, GROUP>();
        constexpr int width = GROUP < 16 ? GROUP : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < count; j++) {
                const int row = drow0 + (offset + j) * rsd.rows_per_it + subd;
                if (row < hidden) yrow[row] = part[j];
            }
        }
    });
    MUMMU_PHASE(5);  // (the end of the kernel: overwrites the mark gate_up_tile left at its own end)
}

// ------------------------------------------------------------------------------------------
// launcher
// ------------------------------------------------------------------------------------------
static int decode_layer_down_iters(const ExpertBanks &b) {
    const RowSplit rs = row_split(b.hidden), rsd = row_split(b.inter);
    const int rpb = kDlWaves * 4 * rs.rows_per_it;
    const int tiles = (b.inter + rpb - 1) / rpb;
    const int per_it = kDlWaves * rsd.rows_per_it * tiles;  // down rows the grid covers per iteration
    return (b.hidden + per_it - 1) / per_it;
}

static bool decode_layer_types(int gate_type, int down_type) {
    return (gate_type == T_Q4_K || gate_type == T_Q8_0) && (down_type == T_Q4_K || down_type == T_Q8_0 || down_type == T_Q6_K);
}

bool decode_layer_supported(const ExpertBanks &b, int k, int n_tokens, const RouterExchange &rx, const LayerExchange &lx) {
    if (!gate_up_fused_supported(b, k, n_tokens, rx)) return false;
    if (k != 8 || b.n_experts > 128) return false;  // one expert slot per XCD; one or two experts per routing lane
    if (b.gate_type != b.up_type || !decode_layer_types(b.gate_type, b.down_type)) return false;
    if (b.inter % 16 != 0 || b.inter > 16 * kActBlocksMax || row_split(b.inter).units > 64) return false;
    if (lx.act_slots == nullptr || lx.y == nullptr || ((uintptr_t)lx.act_slots & 255) != 0) return false;
    return decode_layer_down_iters(b) <= 8;
}

template <int WT, int DT, int NITD, bool EARLY>
static hipError_t launch_decode_layer_t(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                                        int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &ps) {
    const RowSplit rs = row_split(b.hidden);
    const int rpb = kDlWaves * 4 * rs.rows_per_it;
    dim3 grid(k, (b.inter + rpb - 1) / rpb, n_tokens), block(64 * kDlWaves);
    const size_t lds = sizeof(float) * (size_t)rpb + 2 * (size_t)b.hidden + 8 * (size_t)(b.hidden / 16) + 2 * (size_t)b.inter +
                       8 * (size_t)(b.inter / 16);
    if (b.n_experts <= 64)
        launch_kernel(decode_layer_kernel<WT, DT, NITD, 1, EARLY>, grid, block, lds, s, b.gate, b.up, b.down, k, b.hidden, b.inter,
                      b.n_experts, flags, route, rx, lx, ps);
    else
        launch_kernel(decode_layer_kernel<WT, DT, NITD, 2, EARLY>, grid, block, lds, s, b.gate, b.up, b.down, k, b.hidden, b.inter,
                      b.n_experts, flags, route, rx, lx, ps);
    return hipGetLastError();
}

template <int WT, int DT, bool EARLY>
static hipError_t launch_decode_layer_d(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                                        int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &ps) {
    return decode_layer_down_iters(b) <= 4 ? launch_decode_layer_t<WT, DT, 4, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps)
                                           : launch_decode_layer_t<WT, DT, 8, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
}

template <int WT, bool EARLY>
static hipError_t launch_decode_layer_w(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                                        int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &ps) {
    switch (b.down_type) {
    case T_Q4_K: return launch_decode_layer_d<WT, T_Q4_K, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
    case T_Q8_0: return launch_decode_layer_d<WT, T_Q8_0, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
    case T_Q6_K: return launch_decode_layer_d<WT, T_Q6_K, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
    default: return hipErrorInvalidValue;
    }
}

template <bool EARLY>
static hipError_t launch_decode_layer_e(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                                        int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &ps) {
    switch (b.gate_type) {
    case T_Q4_K: return launch_decode_layer_w<T_Q4_K, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
    case T_Q8_0: return launch_decode_layer_w<T_Q8_0, EARLY>(b, rx, lx, route, n_tokens, k, flags, s, ps);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_layer(const ExpertBanks &b, const RouterExchange &rx, const LayerExchange &lx, const RouteInline &route,
                               int n_tokens, int k, int32_t *flags, hipStream_t s, const PendingSum &ps) {
    if (n_tokens <= 0) return hipSuccess;
    if (!decode_layer_supported(b, k, n_tokens, rx, lx)) return hipErrorInvalidValue;
    if (ps.n > 0 && (b.hidden % 256 != 0 || ps.y == nullptr || ps.ids == nullptr || ps.weights == nullptr || ps.out == nullptr ||
                     (((uintptr_t)ps.y | (uintptr_t)ps.residual | (uintptr_t)ps.out) & 15) != 0))
        return hipErrorInvalidValue;
    return b.early_ids ? launch_decode_layer_e<true>(b, rx, lx, route, n_tokens, k, flags, s, ps)
                     : launch_decode_layer_e<false>(b, rx, lx, route, n_tokens, k, flags, s, ps);
}

}  // namespace mummu
