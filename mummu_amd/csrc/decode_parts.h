// Device pieces shared by the decode kernels of block-quantized banks (experts.hip, decode_layer.hip): the gate/up
// products of one workgroup's tile of rows, the exchange of small records between the workgroups of one XCD through
// that XCD's L2, and the prologue that computes router logits, exchanges them and routes the token.
#pragma once

#include "device_utils.h"
#include "kernels.h"
#include "gemv_common.h"
#include "route_common.h"

#include <type_traits>

namespace mummu {

struct NoHook {
    __device__ __forceinline__ void operator()() const {}
    __device__ __forceinline__ void operator()(float) const {}
};

// The gate/up products of one (token, expert) assignment `a` for tile `tile` of output rows, given the
// lane's share `la` of the token's 16-bit activations: NIT iterations of rows_per_it rows per wave, then
// silu(gate) * up per row, written as f32 (act) or staged in LDS (s_act, rows_per_block floats) and - with STORE -
// re-quantized to 16-bit blocks for the down product (ACTQ).  Without STORE the rows are left in s_act and the caller
// goes on after a barrier of its own.  `hook` runs behind the dots of iteration HOOK_AT and is handed one of their
// results: loads whose address it makes depend on that value cannot be asked for before the rows of that iteration have
// arrived (the compiler hoists every independent load to the top of the function, whatever fences lie between).
// `first` runs once the rows of the first iterations have been asked for, in front of every dot.
template <int WT, int UPL, int NIT, bool ACTQ, bool STORE = true, typename Hook = NoHook, int HOOK_AT = NIT - 1, typename First = NoHook>
__device__ __forceinline__ void gate_up_tile(const uint8_t *gate, const uint8_t *up /* (restrict or not is the kernel's choice) */, int e, int a,
                                             const LaneAct<UPL> &la, const RowSplit &rs, int hidden, int inter,
                                             float *__restrict__ act, const QAct &actq, float *s_act, int tile,
                                             Hook hook = Hook(), First first = First()) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane >> rs.group_log2, unit0 = lane & (rs.group - 1);
    const int rows_per_wave = NIT * rs.rows_per_it;
    const int rows_per_block = rows_per_wave * (blockDim.x >> 6);
    const int block_row0 = tile * rows_per_block;
    const int row0 = block_row0 + wave * rows_per_wave;
    const uint32_t row_bytes = (uint32_t)type_row_bytes(WT, hidden);
    const uint8_t *ge = gate + (size_t)uniform_index(e) * (size_t)inter * row_bytes;  // (e is the same in every lane)
    const uint8_t *ue = up + (size_t)uniform_index(e) * (size_t)inter * row_bytes;

    // Software pipeline over the wave's NIT row iterations: the loads of iterations i+1 and i+2
    // are in flight while iteration i is multiplied, so the integer dots run under the stream
    // instead of after it (the scheduling barriers keep the compiler from hoisting every load
    // to the top, where a wave would sit blocked on issue until most of its data had arrived).
    RawRow<WT, UPL> rg[NIT], ru[NIT];
    auto fetch = [&](int i) {
        const int row = row0 + i * rs.rows_per_it + sub;
        const bool ok = row < inter;
        const uint32_t row_off = (uint32_t)(ok ? row : 0) * row_bytes;
        load_row<WT, UPL>(ge, row_off, unit0, rs.units, ok, rg[i]);
        load_row<WT, UPL>(ue, row_off, unit0, rs.units, ok, ru[i]);
    };
    constexpr int AHEAD = NIT < 2 ? NIT : 2;
#pragma unroll
    for (int i = 0; i < AHEAD; i++) fetch(i);
    MUMMU_CODE_FENCE();
    MUMMU_PHASE(1);
    if constexpr (!std::is_same<First, NoHook>::value) {
        first();
        MUMMU_CODE_FENCE();
    }
    float part[2 * NIT];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        if (i + AHEAD < NIT) fetch(i + AHEAD);
        MUMMU_CODE_FENCE();
        part[2 * i] = dot_row<WT, UPL>(rg[i], unit0, la);
        part[2 * i + 1] = dot_row<WT, UPL>(ru[i], unit0, la);
        if (i == HOOK_AT) hook(part[2 * i + 1]);
        MUMMU_CODE_FENCE();
    }
    MUMMU_PHASE(2);
    dispatch_group(rs.group, [&](auto group_tag) {
        constexpr int GROUP = decltype(group_tag)::value;
        constexpr int count = reduced_count<2 * NIT, GROUP>();
        if constexpr (count < 2) {
            // whole-wave rows and fewer than four iterations: the shared reduction would leave a
            // row's gate and up sums in different lanes, so reduce each over the wave instead
#pragma unroll
            for (int i = 0; i < NIT; i++) {
                const float g = wave_sum(part[2 * i]), u = wave_sum(part[2 * i + 1]);
                const int row = row0 + i * rs.rows_per_it + sub;
                if (lane == 0 && row < inter) {
                    const float v = __fmul_rn(det_silu(g), u);
                    if (ACTQ) s_act[row - block_row0] = v;
                    else act[(size_t)a * (size_t)inter + row] = v;
                }
            }
            return;
        }
        const int offset = reduce_partials<2 * NIT, GROUP>(part, lane);
        constexpr int width = GROUP < 16 ? GROUP : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < count; j += 2) {
                const int row = row0 + ((offset + j) >> 1) * rs.rows_per_it + sub;
                if (row < inter) {
                    const float v = __fmul_rn(det_silu(part[j]), part[j + 1]);
                    if (ACTQ) s_act[row - block_row0] = v;
                    else act[(size_t)a * (size_t)inter + row] = v;
                }
            }
        }
    });
    MUMMU_PHASE(3);
    if (ACTQ && STORE) {
        __syncthreads();
        MUMMU_PHASE(4);
        for (int r = threadIdx.x; r < rows_per_block; r += blockDim.x) {
            const int row = block_row0 + r;
            const bool on = row < inter;  // inter % 16 == 0: a 16-lane row is all on or all off
            quantize_store16(on ? s_act[r] : 0.0f, on, actq, (size_t)a, inter, on ? row : 0);
        }
    }
    MUMMU_PHASE(5);
}

// ------------------------------------------------------------------------------------------
// Records passed between the workgroups of one XCD inside a launch.  Producer and consumer sit behind the same L2,
// so a plain 16-byte store followed by a device-scope load (which bypasses the CU's own L1) sees the record within a
// fraction of a microsecond.  A record carries a tag made of the exchange's 64-bit epoch (a device counter that a
// later launch increments), the launch's salt (a host counter: launches that share an epoch - the nodes of one graph
// between two increments - differ in it) and its position, so records of earlier launches never match and a table
// needs no clearing.
// ------------------------------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ inline u32x4 load_device_scope_b128(const u32x4 *p) {
    u32x4 r;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p) : "memory");
    return r;
}

__device__ inline unsigned xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u; }  // HW_REG_XCC_ID[3:0]

__device__ inline u32x4 exchange_record(float logit, unsigned long long epoch, unsigned what) {
    u32x4 r;
    r.x = __float_as_uint(logit);
    r.y = (unsigned)epoch;
    r.z = (unsigned)(epoch >> 32);
    r.w = r.x ^ r.y ^ r.z ^ what ^ 0x5A5A5A5Au;
    return r;
}

// What the `what` of a logit record is made of: its position and the launch's salt.
__device__ inline unsigned logit_what(int t, int n_experts, int row, unsigned salt) {
    return (unsigned)(t * n_experts + row) ^ (salt * 0x9E3779B1u);
}

// Tag of piece `pos` of an activation record (three data words and this tag per 16-byte piece).  For a given
// position the map salt -> tag and the map (low epoch word) -> tag are bijections, so the 2^32 launches before a
// given one all left different tags there.
__device__ inline unsigned act_piece_tag(unsigned long long epoch, unsigned salt, unsigned pos) {
    return ((unsigned)epoch * 0x9E3779B1u) ^ ((unsigned)(epoch >> 32) * 0x85EBCA77u) ^ (salt * 0xC2B2AE3Du) ^ (pos * 0x27D4EB2Fu) ^
           0xA5A5A5A5u;
}

// 8 consecutive activations of one lane (half a 16-element block; the partner lane holds the other half) -> their hi / lo
// bytes, the block's scale and integer sum: the arithmetic of quantize16, bit for bit.
__device__ inline void quantize_half_block(const float (&v)[8], uint2 &hi, uint2 &lo, float &scale, int &sum) {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(v[i]));
    m = fmaxf(m, dpp_move<0xB1>(m));  // the partner lane
    const float inv = m > 0.0f ? __fdiv_rn(32512.0f, m) : 0.0f;
    uint32_t hw[2] = {0u, 0u}, lw[2] = {0u, 0u};
    sum = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        int xq = (int)__builtin_rintf(__fmul_rn(v[i], inv));
        xq = xq > 32512 ? 32512 : (xq < -32512 ? -32512 : xq);
        const int l = ((xq + 128) & 255) - 128;
        const int h = (xq - l) >> 8;
        hw[i >> 2] |= (uint32_t)(h & 255) << (8 * (i & 3));
        lw[i >> 2] |= (uint32_t)(l & 255) << (8 * (i & 3));
        sum += xq;
    }
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, false);
    hi = make_uint2(hw[0], hw[1]);
    lo = make_uint2(lw[0], lw[1]);
    scale = m > 0.0f ? __fdiv_rn(m, 32512.0f) : 0.0f;
}

// load_lane_act from the workgroup's LDS copy of one 16-bit row (UPL = 1: at most 64 units).
template <int WT>
__device__ inline void load_lane_act_lds(const int8_t *s_hi, const int8_t *s_lo, const float *s_scale, const int *s_sum, int unit0,
                                         int units, LaneAct<1> &a) {
    const bool on = unit0 < units;
    int e0, e1;
    unit_halves<WT>(on ? unit0 : 0, e0, e1);
    const int4 h0 = *(const int4 *)(s_hi + e0), h1 = *(const int4 *)(s_hi + e1);
    const int4 l0 = *(const int4 *)(s_lo + e0), l1 = *(const int4 *)(s_lo + e1);
    a.xh[0][0] = h0.x; a.xh[0][1] = h0.y; a.xh[0][2] = h0.z; a.xh[0][3] = h0.w;
    a.xh[0][4] = h1.x; a.xh[0][5] = h1.y; a.xh[0][6] = h1.z; a.xh[0][7] = h1.w;
    a.xl[0][0] = l0.x; a.xl[0][1] = l0.y; a.xl[0][2] = l0.z; a.xl[0][3] = l0.w;
    a.xl[0][4] = l1.x; a.xl[0][5] = l1.y; a.xl[0][6] = l1.z; a.xl[0][7] = l1.w;
    a.s[0][0] = on ? s_scale[e0 >> 4] : 0.0f;
    a.s[0][1] = on ? s_scale[e1 >> 4] : 0.0f;
    a.sx[0][0] = on ? s_sum[e0 >> 4] : 0;
    a.sx[0][1] = on ? s_sum[e1 >> 4] : 0;
    a.fsx[0][0] = __fmul_rn(a.s[0][0], (float)a.sx[0][0]);
    a.fsx[0][1] = __fmul_rn(a.s[0][1], (float)a.sx[0][1]);
}

template <int RT>
__device__ __forceinline__ float router_logit_of(const void *__restrict__ w, int e, const WaveRow &x, int hidden, int lane) {
    WaveRouterRow wr;
    wave_router_row_load<RT>(w, (size_t)e * (size_t)hidden, hidden, lane, wr);
    return wave_router_dot(x, wr, hidden, lane);
}

__device__ __forceinline__ float router_logit_any(const void *__restrict__ w, int wtype, int e, const WaveRow &x, int hidden, int lane) {
    if (wtype == T_F16) return router_logit_of<T_F16>(w, e, x, hidden, lane);
    if (wtype == T_BF16) return router_logit_of<T_BF16>(w, e, x, hidden, lane);
    return router_logit_of<T_F32>(w, e, x, hidden, lane);
}

// ------------------------------------------------------------------------------------------
// The weighted sum over the eight slots of every token of an EARLIER launch, done by a later one: out[t] =
// (residual[t] +) sum over the token's slots in ascending expert id of w * y, multiply and add rounded
// separately - combine_kernel's arithmetic, bit for bit.  One wave takes 64 neighbouring groups of four columns of
// one token (hidden a multiple of 256), wave w_index of w_count.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ void pending_sum_wave(const PendingSum &ps, int hidden, int w_index, int w_count) {
    const int lane = threadIdx.x & 63;
    const int cols4 = hidden >> 2, total = ps.n * cols4;
    for (int base = w_index * 64; base < total; base += w_count * 64) {  // (uniform over the wave)
        const int tp = base / cols4;
        const int col = (base - tp * cols4 + lane) << 2;
        const int my_id = lane < 8 ? ps.ids[(size_t)tp * 8 + lane] : 0x7FFFFFFF;
        const float my_w = lane < 8 ? ps.weights[(size_t)tp * 8 + lane] : 0.0f;
        f32x4 v[8];
#pragma unroll
        for (int s = 0; s < 8; s++) v[s] = *(const f32x4 *)(ps.y + ((size_t)tp * 8 + s) * (size_t)hidden + col);
        f32x4 res = {0.0f, 0.0f, 0.0f, 0.0f};
        if (ps.residual != nullptr) res = *(const f32x4 *)(ps.residual + (size_t)tp * (size_t)hidden + col);
        int rank = 0;  // of slot `lane` by ascending expert id (the ids of one token are distinct; equal ones keep slot order)
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int o = __builtin_amdgcn_readlane(my_id, j);
            rank += (o < my_id) || (o == my_id && j < lane);
        }
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), s));
            v[s].x = __fmul_rn(w, v[s].x);
            v[s].y = __fmul_rn(w, v[s].y);
            v[s].z = __fmul_rn(w, v[s].z);
            v[s].w = __fmul_rn(w, v[s].w);
        }
        int rank_of[8];
#pragma unroll
        for (int s = 0; s < 8; s++) rank_of[s] = __builtin_amdgcn_readlane(rank, s);
        f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int p = 0; p < 8; p++) {
            f32x4 m = v[0];
#pragma unroll
            for (int s = 1; s < 8; s++) m = rank_of[s] == p ? v[s] : m;
            sum.x = __fadd_rn(sum.x, m.x);
            sum.y = __fadd_rn(sum.y, m.y);
            sum.z = __fadd_rn(sum.z, m.z);
            sum.w = __fadd_rn(sum.w, m.w);
        }
        if (ps.residual != nullptr) {
            sum.x = __fadd_rn(res.x, sum.x);
            sum.y = __fadd_rn(res.y, sum.y);
            sum.z = __fadd_rn(res.z, sum.z);
            sum.w = __fadd_rn(res.w, sum.w);
        }
        *(f32x4 *)(ps.out + (size_t)tp * (size_t)hidden + col) = sum;
    }
}

// Reads `warm` (bytes: a multiple of 16) ahead of the launch that will want it, through the L2 of the XCD this workgroup runs on
// (every XCD all of it, as that launch will: read by one XCD only, half of the gain is left): the workgroups of the XCD take a
// slice each, the last wave of each asks for it (shared among all the waves it measured as no read-ahead at all), nobody
// uses the data.  The loads of a pass - four, eight or twelve 16-byte pieces per lane, whichever covers the slice - and the
// wait for them are ONE assembly statement: the compiler never sees a register with a load still on its way into it (it
// would be free to give that register to something else).  The wave that waits here has nothing better to do: the hidden
// row it is about to look for is more than a load's latency away.
__device__ __forceinline__ void warm_next(const void *warm, unsigned bytes) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (warm == nullptr || wave != (int)(blockDim.x >> 6) - 1) return;
    const unsigned per_xcd = (gridDim.x * gridDim.y) >> 3, mine = (blockIdx.y * gridDim.x + blockIdx.x) >> 3;
    const unsigned pieces = bytes >> 4, each = (pieces + per_xcd - 1) / per_xcd;
    const unsigned first = mine * each, end = (mine + 1) * each < pieces ? (mine + 1) * each : pieces;
    if (first >= end) return;
    const u32x4 *base = (const u32x4 *)warm;
    auto at = [&](unsigned i) { return base + (i < end ? i : end - 1); };  // (a piece past the slice's end stands in for its last)
    u32x4 sink;
    for (unsigned i0 = first; i0 < end;) {   // (uniform over the wave)
        const unsigned i = i0 + (unsigned)lane, left = end - i0;
        if (left <= 256u) {
            asm volatile("global_load_dwordx4 %0, %1, off\n\tglobal_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %0, %3, off\n\t"
                         "global_load_dwordx4 %0, %4, off\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(sink) : "v"(at(i)), "v"(at(i + 64)), "v"(at(i + 128)), "v"(at(i + 192)) : "memory");
            i0 += 256;
        } else if (left <= 512u) {
            asm volatile("global_load_dwordx4 %0, %1, off\n\tglobal_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %0, %3, off\n\t"
                         "global_load_dwordx4 %0, %4, off\n\tglobal_load_dwordx4 %0, %5, off\n\tglobal_load_dwordx4 %0, %6, off\n\t"
                         "global_load_dwordx4 %0, %7, off\n\tglobal_load_dwordx4 %0, %8, off\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(sink)
                         : "v"(at(i)), "v"(at(i + 64)), "v"(at(i + 128)), "v"(at(i + 192)), "v"(at(i + 256)), "v"(at(i + 320)), "v"(at(i + 384)),
                           "v"(at(i + 448))
                         : "memory");
            i0 += 512;
        } else {
            asm volatile("global_load_dwordx4 %0, %1, off\n\tglobal_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %0, %3, off\n\t"
                         "global_load_dwordx4 %0, %4, off\n\tglobal_load_dwordx4 %0, %5, off\n\tglobal_load_dwordx4 %0, %6, off\n\t"
                         "global_load_dwordx4 %0, %7, off\n\tglobal_load_dwordx4 %0, %8, off\n\tglobal_load_dwordx4 %0, %9, off\n\t"
                         "global_load_dwordx4 %0, %10, off\n\tglobal_load_dwordx4 %0, %11, off\n\tglobal_load_dwordx4 %0, %12, off\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(sink)
                         : "v"(at(i)), "v"(at(i + 64)), "v"(at(i + 128)), "v"(at(i + 192)), "v"(at(i + 256)), "v"(at(i + 320)), "v"(at(i + 384)),
                           "v"(at(i + 448)), "v"(at(i + 512)), "v"(at(i + 576)), "v"(at(i + 640)), "v"(at(i + 704))
                         : "memory");
            i0 += 768;
        }
    }
}

// LDS a decode workgroup keeps of its token: the 16-bit row of the block's input and the routing.
template <int JN>
struct DecodeShared {
    RouteScratch<JN> route;
    int ids[64];
    float w[64];
    int early_ids[8];  // (EARLY prologue: the eight largest logits, slot order, before the routing proper has run)
};

// What wave 0 of a workgroup carries from the first half of the routing (the logits are in) to the second.
template <int JN>
struct RouteCarry {
    float l[JN];
};

// A finite float as an integer that orders the same way (-0 below +0).
__device__ __forceinline__ int float_order_key(float v) {
    const int b = __float_as_int(v);
    return b ^ ((b >> 31) & 0x7FFFFFFF);
}

// The eight largest of a wave's logits (lane holds experts lane, lane + 64, ...: n_experts <= 64 * JN <= 128), larger first:
// early[s] = the expert of rank s - what the routing picks wherever the probabilities order like the logits.
//
// One expert per lane: every expert counts how many others lie above it.  The keys (the logits as integers that order the
// same way) go through LDS (`stage`, 64 words), every lane reads all of them back with broadcast reads, and an expert
// whose count is below eight writes its own slot: 64 compare-and-add pairs without a cross-lane step, against eight
// dependent wave maxima (0.67 us, measured by running them twice).  So that no two keys are equal, the lowest bits of a
// key give way to the expert's id (the lower id the larger key): two logits closer than 2^7 units in the last place may
// thus come out in the other order than the routing's, one more of the cases its check (route_token_checked8) sends
// through the rounds.  Two experts per lane: eight rounds of the wave maximum, the lower id on equal values (there the
// count, 256 pairs, measured slower: 16.4 against 15.7 us per layer on the 128-expert shape).
template <int JN>
__device__ __forceinline__ void early_top8(const float (&l)[JN], int n_experts, int *early, float *stage) {
    static_assert(JN <= 2, "one or two experts per lane");
    const int lane = threadIdx.x & 63;
    if constexpr (JN == 1) {
        int *keys = (int *)stage;
        const int key = lane < n_experts ? ((float_order_key(l[0]) & ~127) | (127 - lane)) : (int)0x80000000;
        keys[lane] = key;
        wave_lds_sync();
        // (a compare and an add-with-carry per key, four counts side by side so that the adds do not wait for one another)
        int cnt[4] = {0, 0, 0, 0};
        const int4 *kp = (const int4 *)keys;
#pragma unroll
        for (int c = 0; c < 16; c++) {
            const int4 v = kp[c];
            asm("v_cmp_gt_i32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, 0, %0, vcc" : "+v"(cnt[0]) : "v"(v.x), "v"(key) : "vcc");
            asm("v_cmp_gt_i32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, 0, %0, vcc" : "+v"(cnt[1]) : "v"(v.y), "v"(key) : "vcc");
            asm("v_cmp_gt_i32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, 0, %0, vcc" : "+v"(cnt[2]) : "v"(v.z), "v"(key) : "vcc");
            asm("v_cmp_gt_i32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, 0, %0, vcc" : "+v"(cnt[3]) : "v"(v.w), "v"(key) : "vcc");
        }
        const int above = (cnt[0] + cnt[1]) + (cnt[2] + cnt[3]);
        if (above < 8 && lane < n_experts) early[above] = lane;
    } else {
        int cand[JN];
#pragma unroll
        for (int j = 0; j < JN; j++) cand[j] = lane + 64 * j < n_experts ? float_order_key(l[j]) : (int)0x80000000;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            int mine = cand[0];
#pragma unroll
            for (int j = 1; j < JN; j++) mine = cand[j] > mine ? cand[j] : mine;
            const int best = wave_max_i32(mine);
            // lowest expert id holding the maximum: the first lane of the lowest j that has one
            int win = -1;
#pragma unroll
            for (int j = JN - 1; j >= 0; j--) {
                const unsigned long long m = __ballot(cand[j] == best);
                win = m != 0ull ? (int)__builtin_ctzll(m) + 64 * j : win;
            }
#pragma unroll
            for (int j = 0; j < JN; j++) {
                if (lane + 64 * j == win) {
                    early[s] = win;
                    cand[j] = (int)0x80000000;
                }
            }
        }
    }
}

// route_token for k = 8 when the eight winners are believed known (early[0..8), slot order: the eight largest logits):
// the softmax as route_token computes it, then a CHECK that the rounds on the probabilities would pick exactly these
// experts in exactly this order - every slot's probability above the next one's, or equal to it with the lower id, and
// nobody outside as good as the last - instead of the rounds themselves (eight dependent wave maxima), and the
// renormaliser summed in slot order as the rounds would have.  True: ids / weights written, the bits of route_token.
// False (probabilities that tie or cross where the logits do not, a logit that is not finite): nothing written, the
// caller runs route_token.
template <int JN>
__device__ __forceinline__ bool route_token_checked8(const float (&l)[JN], int n_experts, int flavour, int norm, const int *early,
                                                     int32_t *ids, float *weights, RouteScratch<JN> &sc) {
    const int lane = threadIdx.x & 63;
    bool bad = false;
    float mx = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < JN; j++) {
        if (lane + 64 * j < n_experts) {
            bad = bad || !(fabsf(l[j]) <= 3.402823466e38f);
            mx = fmaxf(mx, l[j]);
        }
    }
    if (__any(bad)) return false;
    mx = wave_max(mx);
    float p[JN];
#pragma unroll
    for (int j = 0; j < JN; j++) {
        p[j] = (lane + 64 * j < n_experts) ? det_expf(__fsub_rn(l[j], mx)) : 0.0f;
        sc.p[lane + 64 * j] = p[j];
    }
    wave_lds_sync();
    // (the normaliser: route_token's, line for line)
    const float4 *bp = (const float4 *)sc.p;
    const int chunks = JN == 1 ? 16 : (n_experts + 3) >> 2;
    if (flavour == 0) {
        float total = 0.0f;
#pragma unroll 16
        for (int c = 0; c < chunks; c++) {
            const float4 v = bp[c];
            total = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(total, v.x), v.y), v.z), v.w);
        }
#pragma unroll
        for (int j = 0; j < JN; j++) p[j] = __fdiv_rn(p[j], total);
    } else {
        double total = 0.0;
        bool exact = JN > 1;
#pragma unroll
        for (int j = 0; j < JN; j++) exact = exact && (p[j] == 0.0f || p[j] >= 0x1p-20f);
        if (JN > 1 && __all(exact)) {
#pragma unroll
            for (int j = 0; j < JN; j++) total = __dadd_rn(total, (double)p[j]);
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) total = __dadd_rn(total, __shfl_xor(total, off, 64));
        } else {
#pragma unroll 16
            for (int c = 0; c < chunks; c++) {
                const float4 v = bp[c];
                total = __dadd_rn(__dadd_rn(__dadd_rn(__dadd_rn(total, (double)v.x), (double)v.y), (double)v.z), (double)v.w);
            }
        }
        const float scale = (float)__ddiv_rn(1.0, total);
#pragma unroll
        for (int j = 0; j < JN; j++) p[j] = __fmul_rn(p[j], scale);
    }
    int eid[8];
    float ps[8];
    int my_slot[JN];
#pragma unroll
    for (int j = 0; j < JN; j++) my_slot[j] = -1;
#pragma unroll
    for (int s = 0; s < 8; s++) {
        eid[s] = __builtin_amdgcn_readfirstlane(early[s]);
        float v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[0]), eid[s] & 63));
#pragma unroll
        for (int j = 1; j < JN; j++) {
            const float vj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[j]), eid[s] & 63));
            v = (eid[s] >> 6) == j ? vj : v;
        }
        ps[s] = v;
#pragma unroll
        for (int j = 0; j < JN; j++) my_slot[j] = lane + 64 * j == eid[s] ? s : my_slot[j];
    }
    bool ok = true;
#pragma unroll
    for (int s = 0; s < 7; s++) ok = ok && (ps[s] > ps[s + 1] || (ps[s] == ps[s + 1] && eid[s] < eid[s + 1]));
    bool beats_last = false;
#pragma unroll
    for (int j = 0; j < JN; j++)
        beats_last = beats_last || (lane + 64 * j < n_experts && my_slot[j] < 0 && (p[j] > ps[7] || (p[j] == ps[7] && lane + 64 * j < eid[7])));
    if (!ok || __any(beats_last)) return false;
    float sum32 = 0.0f;
    double sum64 = 0.0;
#pragma unroll
    for (int s = 0; s < 8; s++) {
        sum32 = __fadd_rn(sum32, ps[s]);
        sum64 = __dadd_rn(sum64, (double)ps[s]);
    }
    float denom = 1.0f;
    if (flavour == 0) {
        if (norm) denom = sum32;
    } else {
        const float fs = (float)sum64;
        const float floor_v = 1.0f / 16384.0f;  // experts.rs:74
        denom = fs > floor_v ? fs : floor_v;
    }
#pragma unroll
    for (int j = 0; j < JN; j++) {
        if (my_slot[j] >= 0) {
            float wv = p[j];
            if (flavour != 0 || norm) wv = __fdiv_rn(wv, denom);
            ids[my_slot[j]] = lane + 64 * j;
            weights[my_slot[j]] = wv;
        }
    }
    return true;
}

// Second half of wave 0's routing in the prologue below: the token's logits l -> sh.ids / sh.w in slot order, and, from
// one workgroup per token, the routing, the logits and the hit counters in global memory.  CHECKED: sh.early_ids holds
// the prologue's early pick, which is confirmed where it can be instead of the rounds being run.
template <int JN, bool CHECKED = false>
__device__ __forceinline__ void decode_route_finish(float (&l)[JN], int k, int n_experts, int32_t *__restrict__ flags,
                                                    const RouteInline &route, const RouterExchange &rx, DecodeShared<JN> &sh) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.z;
    if (rx.logits_out != nullptr && blockIdx.x == 0 && blockIdx.y == 0) {
#pragma unroll
        for (int j = 0; j < JN; j++)
            if (lane + 64 * j < n_experts) rx.logits_out[(size_t)t * n_experts + lane + 64 * j] = l[j];
    }
    bool routed = false;
    if constexpr (CHECKED && JN <= 2) routed = route_token_checked8<JN>(l, n_experts, route.flavour, route.norm, sh.early_ids, sh.ids, sh.w, sh.route);
    if (!routed) route_token<JN, false>(l, t, n_experts, k, route.flavour, route.norm, sh.ids, sh.w, nullptr, flags, sh.route, 0);
    wave_lds_sync();
    if (blockIdx.x == 0 && blockIdx.y == 0 && lane < k) {
        const int id = sh.ids[lane];
        route.ids[(size_t)t * k + lane] = id;
        route.weights[(size_t)t * k + lane] = sh.w[lane];
        if (route.hits && (unsigned)id < (unsigned)n_experts) atomicAdd(&route.hits[id], 1ULL);
    }
    MUMMU_PHASE(11);
}

// ------------------------------------------------------------------------------------------
// Prologue of the decode kernels that route by themselves (grid = (slot, row tile, token), four waves per
// workgroup, hidden <= 2048 and a multiple of 64, (slots * row tiles) a multiple of 8).
//
// Workgroups are dealt to the chip's 8 XCDs round-robin by linear id, and the workgroups of one XCD share its L2.
// Those of one token on one XCD split the token's E router rows between them (a wave per row, the fixed summation
// order of router.hip), publish each logit as a 16-byte record in a table of their XCD, and wave 0 of every
// workgroup collects the E records of its XCD before it routes.  The table is indexed by the XCD the workgroup
// actually runs on (read from the hardware id register): a workgroup never looks for records on another XCD.
// The wait is bounded (spin_ticks of the 100 MHz clock): a wave that does not find its records - workgroups placed
// otherwise than assumed, or a tiny spin_ticks from a test - computes the missing logits itself, same bits.
//
// Every wave also loads the token's f32 row: with a gamma it is normalised first (RmsNorm, the RmsNorm kernel's
// bits), wave c quantizes the c-th 512-element chunk to the 16-bit blocks of QAct into LDS (s_xhi, s_xlo, s_xscale,
// s_xsum), which feed the integer dots.  On return the workgroup is past a barrier: sh.ids / sh.w hold the token's
// routing in slot order and the LDS row is complete.  `idle` is called by waves 1.. of the workgroup while wave 0
// routes (they have nothing else to do until the barrier).
// ------------------------------------------------------------------------------------------
//
// EARLY (one expert per routing lane, k = 8): wave 0 stops once it has the logits and the eight LARGEST OF THEM in
// sh.early_ids - the experts the routing will pick wherever the probabilities order like the logits, which softmax all
// but guarantees - and the workgroup goes on with those; wave 0 runs the routing proper later, through
// decode_route_finish, behind its first row loads (the softmax, the rounds on probabilities and the renormalisation are
// some 350 dependent instructions that no expert byte had been asked for until now).  The caller compares sh.ids with
// what it started on and starts over where they differ (two logits whose probabilities round to the same float, or
// cross: a tie goes to the lower id, not to the larger logit).
template <int JN, typename Idle = NoHook, bool EARLY = false>
__device__ __forceinline__ unsigned long long decode_route_prologue(int k, int hidden, int n_experts, int32_t *__restrict__ flags,
                                                                    const RouteInline &route, const RouterExchange &rx,
                                                                    DecodeShared<JN> &sh, int8_t *s_xhi, int8_t *s_xlo,
                                                                    float *s_xscale, int *s_xsum, Idle idle = Idle(),
                                                                    RouteCarry<JN> *carry = nullptr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.z;

    // which router rows this workgroup computes: the workgroups of token t on one XCD are those with the same linear id
    // modulo 8; `mine` counts them in linear order
    const int per_token = gridDim.x * gridDim.y;             // a multiple of 8
    const int per_xcd = per_token >> 3;
    const int mine = (blockIdx.y * gridDim.x + blockIdx.x) >> 3;
    const int rows_each = (n_experts + per_xcd - 1) / per_xcd;
    const int row_begin = mine * rows_each;
    const int row_end = row_begin + rows_each < n_experts ? row_begin + rows_each : n_experts;

    // every load that does not depend on anything goes out first: the epoch, the token's row, this wave's router row.
    // A wave with a router row (or with a gamma: the sum of squares runs over the whole row) and wave 0 take the whole row,
    // the others only the 512-element chunk they quantize (chunk = wave: four waves, at most four chunks).
    const unsigned long long epoch = *rx.epoch;
    const float *xr = rx.x + (size_t)t * (size_t)hidden;
    const int my_row = row_begin + wave, my_end = row_end;
    const bool whole_row = rx.gamma != nullptr || my_row < my_end || wave == 0;  // (wave 0: it may have to compute missing logits)
    const int qbase = lane * 8 + 512 * wave;
    const bool qon = qbase < hidden;  // hidden % 64 == 0: the two lanes of a 16-element block are on or off together
    WaveRow xrow;
    f32x4 qa, qb;
    if (whole_row) {
        wave_row_load(xr, hidden, lane, xrow);
    } else {
        qa = ((const f32x4 *)(xr + (qon ? qbase : 0)))[0];
        qb = ((const f32x4 *)(xr + (qon ? qbase : 0)))[1];
    }
    WaveRouterRow wrow;
    if (my_row < my_end) {
        const size_t at = (size_t)my_row * (size_t)hidden;
        if (rx.wtype == T_F16) wave_router_row_load<T_F16>(rx.w, at, hidden, lane, wrow);
        else if (rx.wtype == T_BF16) wave_router_row_load<T_BF16>(rx.w, at, hidden, lane, wrow);
        else wave_router_row_load<T_F32>(rx.w, at, hidden, lane, wrow);
    }
    if (rx.gamma != nullptr) {
        const float r = wave_row_rms_scale(xrow, hidden, lane, rx.eps);
        wave_row_normalise(xrow, r, rx.gamma, hidden, lane);
        if (rx.xnorm_out != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && wave == 0) {
            float *xo = rx.xnorm_out + (size_t)t * (size_t)hidden;
#pragma unroll
            for (int c = 0; c < kWaveRowChunks; c++) {
                const int base = lane * 8 + 512 * c;
                if (base >= hidden) continue;
                ((f32x4 *)(xo + base))[0] = xrow.a[c];
                ((f32x4 *)(xo + base))[1] = xrow.b[c];
            }
        }
    }
    u32x4 *table = (u32x4 *)rx.slots + ((size_t)xcc_id() * kExchangeTokens + (size_t)t) * (size_t)n_experts;
    // this wave's router row (more rows than waves: the remaining ones in further rounds, each with its own loads)
    if (my_row < my_end) {
        const float logit = wave_router_dot(xrow, wrow, hidden, lane);
        if (lane == 0) table[my_row] = exchange_record(logit, epoch, logit_what(t, n_experts, my_row, rx.salt));
    }
    for (int row = row_begin + wave + (blockDim.x >> 6); row < row_end; row += blockDim.x >> 6) {
        const float logit = router_logit_any(rx.w, rx.wtype, row, xrow, hidden, lane);
        if (lane == 0) table[row] = exchange_record(logit, epoch, logit_what(t, n_experts, row, rx.salt));
    }
    MUMMU_PHASE(8);
    // this wave's chunk of the row into LDS as 16-bit blocks (lane pairs hold the 16-element blocks)
    if (whole_row) {
        qa = xrow.a[0];
        qb = xrow.b[0];
#pragma unroll
        for (int cc = 1; cc < kWaveRowChunks; cc++) {
            qa = wave == cc ? xrow.a[cc] : qa;
            qb = wave == cc ? xrow.b[cc] : qb;
        }
    }
    if (512 * wave < hidden) {
        const float v[8] = {qon ? qa.x : 0.0f, qon ? qa.y : 0.0f, qon ? qa.z : 0.0f, qon ? qa.w : 0.0f,
                            qon ? qb.x : 0.0f, qon ? qb.y : 0.0f, qon ? qb.z : 0.0f, qon ? qb.w : 0.0f};
        uint2 hi, lo;
        float scale;
        int sum;
        quantize_half_block(v, hi, lo, scale, sum);
        if (qon) {
            *(uint2 *)(s_xhi + qbase) = hi;
            *(uint2 *)(s_xlo + qbase) = lo;
            if ((lane & 1) == 0) {
                s_xscale[qbase >> 4] = scale;
                s_xsum[qbase >> 4] = sum;
            }
            if (rx.xq_out.hi != nullptr && blockIdx.x == 0 && blockIdx.y == 0) {
                // one workgroup per token also leaves the row in global memory (the shared expert's launches read it)
                *(uint2 *)(rx.xq_out.hi + (size_t)t * (size_t)hidden + qbase) = hi;
                *(uint2 *)(rx.xq_out.lo + (size_t)t * (size_t)hidden + qbase) = lo;
                if ((lane & 1) == 0) {
                    rx.xq_out.scale[(size_t)t * (size_t)(hidden / 16) + (qbase >> 4)] = scale;
                    rx.xq_out.sum[(size_t)t * (size_t)(hidden / 16) + (qbase >> 4)] = sum;
                }
            }
        }
    }
    MUMMU_PHASE(9);
    if (wave == 0) {
        // collect the E logits of token t from this XCD's table
        float l[JN];
        bool have[JN];
#pragma unroll
        for (int j = 0; j < JN; j++) {
            l[j] = 0.0f;
            have[j] = lane + 64 * j >= n_experts;
        }
        const unsigned long long t_begin = wall_clock64();
        bool complete = false;
        while (rx.spin_ticks != 0u) {  // (a bound of 0: do not look at the table at all)
            bool all = true;
#pragma unroll
            for (int j = 0; j < JN; j++) {
                if (have[j]) continue;
                const int e = lane + 64 * j;
                const u32x4 r = load_device_scope_b128(table + e);
                const u32x4 want = exchange_record(__uint_as_float(r.x), epoch, logit_what(t, n_experts, e, rx.salt));
                if (r.y == want.y && r.z == want.z && r.w == want.w) {
                    l[j] = __uint_as_float(r.x);
                    have[j] = true;
                } else {
                    all = false;
                }
            }
            if (__all(all)) {
                complete = true;
                break;
            }
            if (wall_clock64() - t_begin >= (unsigned long long)rx.spin_ticks) break;
            __builtin_amdgcn_s_sleep(1);
        }
        MUMMU_PHASE(10);
        if (!complete) {
            // records that never came: compute those logits here (the same function of the same row: the same bits)
            if (lane == 0 && rx.fallbacks != nullptr) atomicAdd(rx.fallbacks, 1ULL);
#pragma unroll
            for (int j = 0; j < JN; j++) {
                unsigned long long missing = __ballot(!have[j]);
                while (missing != 0ull) {
                    const int src = (int)__builtin_ctzll(missing);
                    missing &= missing - 1ull;
                    const float v = router_logit_any(rx.w, rx.wtype, src + 64 * j, xrow, hidden, lane);
                    if (lane == src) l[j] = v;
                }
            }
        }
        if constexpr (EARLY) {
            static_assert(JN <= 2, "one or two experts per routing lane");
            early_top8<JN>(l, n_experts, sh.early_ids, sh.route.p);
#pragma unroll
            for (int j = 0; j < JN; j++) carry->l[j] = l[j];
            MUMMU_PHASE(11);
        } else {
            decode_route_finish<JN>(l, k, n_experts, flags, route, rx, sh);
        }
    } else {
        idle();
    }
    __syncthreads();
    MUMMU_PHASE(7);
    return epoch;
}

}  // namespace mummu
