// SwiGLU expert products for small batches (decode): packed GEMV straight off the GGUF bytes
// resident in HBM, plus the weighted combine.
//
// Reference semantics: down(silu(gate.x) * (up.x)) per routed (token, expert) pair
// (nn/moe.rs:312-316, models/qwen4exp/experts.rs:781-845), results scatter-added in
// ascending expert id with two roundings (nn/moe.rs:1590-1601, experts.rs:1137-1148).
//
// Work decomposition: blockIdx.x = one (token, expert) assignment a = t*k + s, blockIdx.y = a
// tile of output rows.  A wave walks its rows; the lanes of a wave split one weight row in
// 16-byte units (Q4_K: one 16-byte slice of a super-block's nibbles; Q8_0: one 34-byte
// block; float types: consecutive elements), so every global load is a contiguous run.
//
// Arithmetic of the quantized types (Q4_K, Q8_0): the activation row is quantized ONCE per
// wave, in registers, to 16-bit integers xq = rint(x * 32512/amax) with one f32 scale
// s = amax/32512 per activation block (64 elements under Q4_K - one low/high nibble chunk -
// and 32 under Q8_0), split into two signed bytes xq = 256*hi + lo.  Weight codes and
// activation bytes meet in v_dot4_i32_i8, so the block sums  sum(q * xq)  are exact integers;
// only the scale products are floating point:
//     Q8_0 block :              d * (s * float(sum q*xq))
//     Q4_K sub-block pair:  (d*s) * float(sc0*sum(q0*xq0) + sc1*sum(q1*xq1))
//                         - (dmin*s) * float(m0*sum(xq0) + m1*sum(xq1))
// A 16-bit activation is ~2^-15 of the block maximum - about 100x finer than the int8
// activations llama.cpp multiplies these formats with - and, being a function of the token's
// own row only, keeps the result independent of how many tokens share the call.
// Float weight types (F32/F16/BF16) run an f32 fma chain per lane on the exact f32 value of
// each weight.
#include "device_utils.h"
#include "kernels.h"

namespace mummu {

constexpr int kGemvWaves = 4;  // waves per workgroup

// ------------------------------------------------------------------------------------------
// Lane geometry of one weight row split in "units" (see file comment).
// ------------------------------------------------------------------------------------------
struct RowSplit {
    int units;        // units per row
    int group;        // lanes that share a row (power of two, <= 64)
    int rows_per_it;  // rows a wave handles per iteration = 64 / group
};

__host__ __device__ inline RowSplit row_split(int type, int in_dim) {
    RowSplit r;
    r.units = type == T_Q4_K ? in_dim / 32 : in_dim / 32;  // Q4_K: 8 units per 256; Q8_0: 1 per 32
    int g = 1;
    while (g < r.units && g < 64) g <<= 1;
    r.group = g;
    r.rows_per_it = 64 / g;
    return r;
}

template <int UPL>
struct LaneAct {
    int xh[UPL][8];  // hi bytes of the lane's 32 activations, 4 per word
    int xl[UPL][8];  // lo bytes
    float s[UPL];    // scale of the activation block the lane's 32 elements belong to
    int sx[UPL][2];  // sum(xq) over the first / second 16 elements (Q4_K min term)
};

// Start elements of the two 16-element halves unit u of a row covers.
template <int WT>
__device__ inline void unit_halves(int u, int &e0, int &e1) {
    if constexpr (WT == T_Q4_K) {
        int sb = u >> 3, up = u & 7;
        e0 = sb * 256 + (up >> 1) * 64 + (up & 1) * 16;  // low nibbles: elements of sub-block 2c
        e1 = e0 + 32;                                    // high nibbles: sub-block 2c+1
    } else {
        e0 = u * 32;
        e1 = e0 + 16;
    }
}

__device__ inline void quantize16(const float (&v)[16], float inv, int *xh, int *xl, int &sum) {
    sum = 0;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t hw = 0, lw = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int q = (int)__builtin_rintf(__fmul_rn(v[4 * w + j], inv));
            q = q > 32512 ? 32512 : (q < -32512 ? -32512 : q);
            int lo = ((q + 128) & 255) - 128;
            int hi = (q - lo) >> 8;
            sum += q;
            hw |= ((uint32_t)hi & 0xFFu) << (8 * j);
            lw |= ((uint32_t)lo & 0xFFu) << (8 * j);
        }
        xh[w] = (int)hw;
        xl[w] = (int)lw;
    }
}

// Quantize the lane's share of activation row `xrow` (f32, in_dim wide).  The activation
// block (one scale) is the 64-element chunk for Q4_K - the lane's two halves plus those of the
// neighbouring unit, lane ^ 1 - and the 32-element block for Q8_0.
template <int WT, int UPL>
__device__ inline void load_lane_act(const float *__restrict__ xrow, int unit0, int units, LaneAct<UPL> &a) {
#pragma unroll
    for (int i = 0; i < UPL; i++) {
        int u = unit0 + 64 * i;
        bool on = u < units;
        int e0, e1;
        unit_halves<WT>(on ? u : 0, e0, e1);
        float v0[16], v1[16];
        const float4 *p0 = (const float4 *)(xrow + e0);
        const float4 *p1 = (const float4 *)(xrow + e1);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float4 a0 = p0[j], a1 = p1[j];
            v0[4 * j] = a0.x; v0[4 * j + 1] = a0.y; v0[4 * j + 2] = a0.z; v0[4 * j + 3] = a0.w;
            v1[4 * j] = a1.x; v1[4 * j + 1] = a1.y; v1[4 * j + 2] = a1.z; v1[4 * j + 3] = a1.w;
        }
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; j++) m = fmaxf(m, fmaxf(fabsf(v0[j]), fabsf(v1[j])));
        if (!on) m = 0.0f;
        if constexpr (WT == T_Q4_K) m = fmaxf(m, dpp_move<0xB1>(m));  // lane ^ 1 holds the rest of the chunk
        const float inv = m > 0.0f ? __fdiv_rn(32512.0f, m) : 0.0f;
        a.s[i] = m > 0.0f ? __fdiv_rn(m, 32512.0f) : 0.0f;
        quantize16(v0, inv, &a.xh[i][0], &a.xl[i][0], a.sx[i][0]);
        quantize16(v1, inv, &a.xh[i][4], &a.xl[i][4], a.sx[i][1]);
        if (!on) {
#pragma unroll
            for (int w = 0; w < 8; w++) a.xh[i][w] = a.xl[i][w] = 0;
            a.s[i] = 0.0f;
            a.sx[i][0] = a.sx[i][1] = 0;
        }
    }
}

// The lane's raw share of one quantized weight row, as loaded (nothing decoded yet), so that a
// wave can put the loads of several rows in flight before it touches any of them.
template <int WT, int UPL>
struct RawRow;
template <int UPL>
struct RawRow<T_Q4_K, UPL> {
    uint4 hdr[UPL];  // f16 d, f16 dmin, 12 B of 6-bit scales/mins
    uint4 q[UPL];    // the lane's 16 bytes of nibbles
};
template <int UPL>
struct RawRow<T_Q8_0, UPL> {
    uint32_t d[UPL];     // f16 scale bits
    uint32_t q[UPL][8];  // 32 int8 codes
};

template <int WT, int UPL>
__device__ inline void load_row(const uint8_t *__restrict__ rowp, int unit0, int units, bool ok, RawRow<WT, UPL> &r) {
#pragma unroll
    for (int i = 0; i < UPL; i++) {
        const int u = unit0 + 64 * i;
        const bool on = ok && u < units;
        if constexpr (WT == T_Q4_K) {
            r.hdr[i] = make_uint4(0, 0, 0, 0);
            r.q[i] = make_uint4(0, 0, 0, 0);
            if (on) {
                const uint8_t *blk = rowp + (size_t)(u >> 3) * 144;
                r.hdr[i] = *(const uint4 *)blk;
                r.q[i] = *(const uint4 *)(blk + 16 + (u & 7) * 16);
            }
        } else {
            r.d[i] = 0;
#pragma unroll
            for (int w = 0; w < 8; w++) r.q[i][w] = 0;
            if (on) {
                const uint8_t *blk = rowp + (size_t)u * 34;
                uint16_t db;
                __builtin_memcpy(&db, blk, 2);
                r.d[i] = db;
#pragma unroll
                for (int w = 0; w < 8; w++) __builtin_memcpy(&r.q[i][w], blk + 2 + 4 * w, 4);  // 2-byte aligned
            }
        }
    }
}

// The lane's partial of <row, activation>.  A lane that loaded nothing holds zero scales and
// contributes exactly 0.
//   Q4_K: with q the 4-bit codes, xq the 16-bit activations of the lane's two 16-element halves
//   (sub-blocks 2c and 2c+1 of one super-block, one activation scale s),
//       (d*s) * float(sc0*sum(q0*xq0) + sc1*sum(q1*xq1)) - (dmin*s) * float(m0*sum(xq0) + m1*sum(xq1))
//   where every sum and both 6-bit-weighted combinations are exact integers.
//   Q8_0: d * (s * float(sum(q*xq))).
template <int WT, int UPL>
__device__ inline float dot_row(const RawRow<WT, UPL> &r, int unit0, const LaneAct<UPL> &a) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < UPL; i++) {
        if constexpr (WT == T_Q4_K) {
            const int u = unit0 + 64 * i;
            const uint4 hdr = r.hdr[i];
            const float d = half_bits_to_float((uint16_t)(hdr.x & 0xFFFFu));
            const float dmin = half_bits_to_float((uint16_t)(hdr.x >> 16));
            // 6-bit (scale, min) of sub-blocks 2c, 2c+1 (ggml get_scale_min_k4), c fixed per lane
            const int c = (u & 7) >> 1;
            const int sh = 16 * (c & 1);
            int sc0, sc1, mn0, mn1;
            if (c < 2) {
                sc0 = (int)((hdr.y >> sh) & 63u);
                sc1 = (int)((hdr.y >> (sh + 8)) & 63u);
                mn0 = (int)((hdr.z >> sh) & 63u);
                mn1 = (int)((hdr.z >> (sh + 8)) & 63u);
            } else {
                const uint32_t lo = hdr.w >> sh;
                sc0 = (int)((lo & 0xFu) | (((hdr.y >> (sh + 6)) & 3u) << 4));
                mn0 = (int)(((lo >> 4) & 0xFu) | (((hdr.z >> (sh + 6)) & 3u) << 4));
                sc1 = (int)(((lo >> 8) & 0xFu) | (((hdr.y >> (sh + 14)) & 3u) << 4));
                mn1 = (int)(((lo >> 12) & 0xFu) | (((hdr.z >> (sh + 14)) & 3u) << 4));
            }
            const uint32_t q[4] = {r.q[i].x, r.q[i].y, r.q[i].z, r.q[i].w};
            int lh = 0, ll = 0, hh = 0, hl = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                int lo = (int)(q[w] & 0x0F0F0F0Fu);
                int hi = (int)((q[w] >> 4) & 0x0F0F0F0Fu);
                lh = __builtin_amdgcn_sdot4(lo, a.xh[i][w], lh, false);
                ll = __builtin_amdgcn_sdot4(lo, a.xl[i][w], ll, false);
                hh = __builtin_amdgcn_sdot4(hi, a.xh[i][4 + w], hh, false);
                hl = __builtin_amdgcn_sdot4(hi, a.xl[i][4 + w], hl, false);
            }
            // |sum(q*xq)| <= 15*32512*16 < 2^23 and |sum(xq)| <= 16*32512: 24-bit multiplies are exact
            const int pos = __mul24(sc0, lh * 256 + ll) + __mul24(sc1, hh * 256 + hl);
            const int neg = __mul24(mn0, a.sx[i][0]) + __mul24(mn1, a.sx[i][1]);
            const float t = __fmul_rn(__fmul_rn(d, a.s[i]), (float)pos);
            acc = __fadd_rn(acc, __builtin_fmaf(-__fmul_rn(dmin, a.s[i]), (float)neg, t));
        } else {  // Q8_0
            float d = half_bits_to_float((uint16_t)r.d[i]);
            int sh = 0, sl = 0;
#pragma unroll
            for (int w = 0; w < 8; w++) {
                sh = __builtin_amdgcn_sdot4((int)r.q[i][w], a.xh[i][w], sh, false);
                sl = __builtin_amdgcn_sdot4((int)r.q[i][w], a.xl[i][w], sl, false);
            }
            float t = __fmul_rn((float)(sh * 256 + sl), a.s[i]);
            acc = __builtin_fmaf(d, t, acc);
        }
    }
    return acc;
}

// The lane's partial of <row, activation> for a float row: elements lane*VEC + 64*VEC*j.
template <int WT, int VEC>
__device__ inline float row_partial_f(const uint8_t *__restrict__ rowp, const float *__restrict__ xrow, int in_dim,
                                      int lane) {
    float acc = 0.0f;
    for (int i = lane * VEC; i < in_dim; i += 64 * VEC) {
        float w[VEC];
        if constexpr (WT == T_F32) {
            if constexpr (VEC == 4) {
                float4 v = *(const float4 *)(rowp + (size_t)i * 4);
                w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
            } else {
                w[0] = *(const float *)(rowp + (size_t)i * 4);
            }
        } else {
            if constexpr (VEC == 4) {
                uint2 v = *(const uint2 *)(rowp + (size_t)i * 2);
                uint16_t h[4] = {(uint16_t)(v.x & 0xFFFF), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xFFFF), (uint16_t)(v.y >> 16)};
#pragma unroll
                for (int j = 0; j < 4; j++) w[j] = WT == T_F16 ? half_bits_to_float(h[j]) : bf16_bits_to_float(h[j]);
            } else {
                uint16_t h = *(const uint16_t *)(rowp + (size_t)i * 2);
                w[0] = WT == T_F16 ? half_bits_to_float(h) : bf16_bits_to_float(h);
            }
        }
        if constexpr (VEC == 4) {
            float4 xv = *(const float4 *)(xrow + i);
            acc = __builtin_fmaf(w[0], xv.x, acc);
            acc = __builtin_fmaf(w[1], xv.y, acc);
            acc = __builtin_fmaf(w[2], xv.z, acc);
            acc = __builtin_fmaf(w[3], xv.w, acc);
        } else {
            acc = __builtin_fmaf(w[0], xrow[i], acc);
        }
    }
    return acc;
}

__host__ __device__ inline size_t type_row_bytes(int type, int in_dim) {
    return (size_t)(in_dim / block_elems(type)) * (size_t)block_bytes(type);
}

// ------------------------------------------------------------------------------------------
// gate/up: act[a, j] = silu(<gate_e[j], x_t>) * <up_e[j], x_t>
// ------------------------------------------------------------------------------------------
template <int WT, int UPL, int VEC, int NIT>
__global__ __launch_bounds__(64 * kGemvWaves) void gate_up_kernel(
    const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up, const float *__restrict__ x,
    const int32_t *__restrict__ ids, int k, int fixed_expert, int hidden, int inter, int n_experts,
    int rows_per_wave, float *__restrict__ act, int32_t *__restrict__ flags) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = blockIdx.x;
    const int e = fixed_expert >= 0 ? fixed_expert : ids[a];
    const int t = fixed_expert >= 0 ? a : a / k;
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

    if constexpr (WT == T_Q4_K || WT == T_Q8_0) {
        // rows_per_wave == NIT * rows_per_it: every weight load of the wave is issued before
        // the first one is consumed
        const RowSplit rs = row_split(WT, hidden);
        const int sub = lane / rs.group, unit0 = lane % rs.group;
        LaneAct<UPL> la;
        load_lane_act<WT, UPL>(xrow, unit0, rs.units, la);
        RawRow<WT, UPL> rg[NIT], ru[NIT];
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            const int row = row0 + i * rs.rows_per_it + sub;
            const bool ok = row < inter;
            load_row<WT, UPL>(ge + (size_t)(ok ? row : 0) * row_bytes, unit0, rs.units, ok, rg[i]);
            load_row<WT, UPL>(ue + (size_t)(ok ? row : 0) * row_bytes, unit0, rs.units, ok, ru[i]);
        }
        float part[2 * NIT];
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            part[2 * i] = dot_row<WT, UPL>(rg[i], unit0, la);
            part[2 * i + 1] = dot_row<WT, UPL>(ru[i], unit0, la);
        }
        int count, offset;
        reduce_partials<2 * NIT>(part, rs.group, lane, count, offset);
        const int width = rs.group < 16 ? rs.group : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < 2 * NIT; j += 2) {
                if (j < count) {
                    const int row = row0 + ((offset + j) >> 1) * rs.rows_per_it + sub;
                    if (row < inter) arow[row] = __fmul_rn(det_silu(part[j]), part[j + 1]);
                }
            }
        }
    } else {
        for (int r = 0; r < rows_per_wave; r++) {
            const int row = row0 + r;
            if (row >= inter) break;
            float pg = row_partial_f<WT, VEC>(ge + (size_t)row * row_bytes, xrow, hidden, lane);
            float pu = row_partial_f<WT, VEC>(ue + (size_t)row * row_bytes, xrow, hidden, lane);
            pg = wave_sum(pg);
            pu = wave_sum(pu);
            if (lane == 0) arow[row] = __fmul_rn(det_silu(pg), pu);
        }
    }
}

// ------------------------------------------------------------------------------------------
// down: y[a, c] = <down_e[c], act[a]>
// ------------------------------------------------------------------------------------------
template <int WT, int UPL, int VEC, int NIT>
__global__ __launch_bounds__(64 * kGemvWaves) void down_kernel(const uint8_t *__restrict__ down,
                                                               const float *__restrict__ act,
                                                               const int32_t *__restrict__ ids, int fixed_expert,
                                                               int hidden, int inter, int n_experts, int rows_per_wave,
                                                               float *__restrict__ y) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = blockIdx.x;
    const int e = fixed_expert >= 0 ? fixed_expert : ids[a];
    if ((unsigned)e >= (unsigned)n_experts) return;  // flagged by gate_up
    const size_t row_bytes = type_row_bytes(WT, inter);
    const uint8_t *de = down + (size_t)e * (size_t)hidden * row_bytes;
    const float *arow = act + (size_t)a * (size_t)inter;
    float *yrow = y + (size_t)a * (size_t)hidden;
    const int row0 = (blockIdx.y * kGemvWaves + wave) * rows_per_wave;

    if constexpr (WT == T_Q4_K || WT == T_Q8_0) {
        const RowSplit rs = row_split(WT, inter);
        const int sub = lane / rs.group, unit0 = lane % rs.group;
        RawRow<WT, UPL> rd[NIT];
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            const int row = row0 + i * rs.rows_per_it + sub;
            const bool ok = row < hidden;
            load_row<WT, UPL>(de + (size_t)(ok ? row : 0) * row_bytes, unit0, rs.units, ok, rd[i]);
        }
        LaneAct<UPL> la;
        load_lane_act<WT, UPL>(arow, unit0, rs.units, la);
        float part[NIT];
#pragma unroll
        for (int i = 0; i < NIT; i++) part[i] = dot_row<WT, UPL>(rd[i], unit0, la);
        int count, offset;
        reduce_partials<NIT>(part, rs.group, lane, count, offset);
        const int width = rs.group < 16 ? rs.group : 16;
        if ((lane & (width - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < NIT; j++) {
                if (j < count) {
                    const int row = row0 + (offset + j) * rs.rows_per_it + sub;
                    if (row < hidden) yrow[row] = part[j];
                }
            }
        }
    } else {
        for (int r = 0; r < rows_per_wave; r++) {
            const int row = row0 + r;
            if (row >= hidden) break;
            float p = row_partial_f<WT, VEC>(de + (size_t)row * row_bytes, arow, inter, lane);
            p = wave_sum(p);
            if (lane == 0) yrow[row] = p;
        }
    }
}

// Float rows: rows per wave so that a launch has a few thousand waves without tiny tiles.
static int pick_rows_per_wave(int out_dim, int n_assign) {
    int rpw = 1;
    while ((long)((out_dim + rpw * 2 - 1) / (rpw * 2)) * n_assign >= 4096 && rpw < 64) rpw *= 2;
    return rpw < 4 ? 4 : rpw;
}

// Quantized rows: NIT iterations of rows_per_it rows per wave, all loads in flight at once.
// NIT shrinks as units-per-lane grows so the raw rows stay in registers.
template <int WT>
static hipError_t launch_gate_up_t(const ExpertBanks &b, const float *x, const int32_t *ids, int n_assign, int k,
                                   int fixed_expert, float *act, int32_t *flags, hipStream_t s) {
    constexpr bool quant = WT == T_Q4_K || WT == T_Q8_0;
    dim3 block(64 * kGemvWaves);
#define MUMMU_GU(UPL, VEC, NIT, RPW)                                                                                \
    do {                                                                                                            \
        const int rpw_ = (RPW);                                                                                     \
        dim3 grid(n_assign, (b.inter + rpw_ * kGemvWaves - 1) / (rpw_ * kGemvWaves));                               \
        gate_up_kernel<WT, UPL, VEC, NIT><<<grid, block, 0, s>>>(b.gate, b.up, x, ids, k, fixed_expert, b.hidden,   \
                                                                 b.inter, b.n_experts, rpw_, act, flags);           \
    } while (0)
    if constexpr (quant) {
        const RowSplit rs = row_split(WT, b.hidden);
        const int upl = (rs.units + 63) / 64;
        if (upl == 1) MUMMU_GU(1, 1, 4, 4 * rs.rows_per_it);
        else if (upl == 2) MUMMU_GU(2, 1, 2, 2 * rs.rows_per_it);
        else if (upl <= 4) MUMMU_GU(4, 1, 1, rs.rows_per_it);
        else return hipErrorInvalidValue;
    } else {
        const int rpw = pick_rows_per_wave(b.inter, n_assign);
        const bool vec = b.hidden % 4 == 0 && (((uintptr_t)x & 15) == 0);
        if (vec) MUMMU_GU(1, 4, 1, rpw);
        else MUMMU_GU(1, 1, 1, rpw);
    }
#undef MUMMU_GU
    return hipGetLastError();
}

hipError_t launch_gate_up(const ExpertBanks &b, const float *x, const int32_t *ids, int n_assign, int k,
                          int fixed_expert, float *act, int32_t *flags, hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    if (b.gate_type != b.up_type) return hipErrorInvalidValue;
    switch (b.gate_type) {
    case T_F32: return launch_gate_up_t<T_F32>(b, x, ids, n_assign, k, fixed_expert, act, flags, s);
    case T_F16: return launch_gate_up_t<T_F16>(b, x, ids, n_assign, k, fixed_expert, act, flags, s);
    case T_BF16: return launch_gate_up_t<T_BF16>(b, x, ids, n_assign, k, fixed_expert, act, flags, s);
    case T_Q8_0: return launch_gate_up_t<T_Q8_0>(b, x, ids, n_assign, k, fixed_expert, act, flags, s);
    case T_Q4_K: return launch_gate_up_t<T_Q4_K>(b, x, ids, n_assign, k, fixed_expert, act, flags, s);
    default: return hipErrorInvalidValue;
    }
}

template <int WT>
static hipError_t launch_down_t(const ExpertBanks &b, const float *act, const int32_t *ids, int n_assign,
                                int fixed_expert, float *y, hipStream_t s) {
    constexpr bool quant = WT == T_Q4_K || WT == T_Q8_0;
    dim3 block(64 * kGemvWaves);
#define MUMMU_DN(UPL, VEC, NIT, RPW)                                                                                \
    do {                                                                                                            \
        const int rpw_ = (RPW);                                                                                     \
        dim3 grid(n_assign, (b.hidden + rpw_ * kGemvWaves - 1) / (rpw_ * kGemvWaves));                              \
        down_kernel<WT, UPL, VEC, NIT><<<grid, block, 0, s>>>(b.down, act, ids, fixed_expert, b.hidden, b.inter,    \
                                                              b.n_experts, rpw_, y);                                \
    } while (0)
    if constexpr (quant) {
        const RowSplit rs = row_split(WT, b.inter);
        const int upl = (rs.units + 63) / 64;
        if (upl == 1) MUMMU_DN(1, 1, 4, 4 * rs.rows_per_it);
        else if (upl == 2) MUMMU_DN(2, 1, 2, 2 * rs.rows_per_it);
        else if (upl <= 4) MUMMU_DN(4, 1, 1, rs.rows_per_it);
        else return hipErrorInvalidValue;
    } else {
        const int rpw = pick_rows_per_wave(b.hidden, n_assign);
        if (b.inter % 4 == 0) MUMMU_DN(1, 4, 1, rpw);
        else MUMMU_DN(1, 1, 1, rpw);
    }
#undef MUMMU_DN
    return hipGetLastError();
}

hipError_t launch_down(const ExpertBanks &b, const float *act, const int32_t *ids, int n_assign, int fixed_expert,
                       float *y, hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    switch (b.down_type) {
    case T_F32: return launch_down_t<T_F32>(b, act, ids, n_assign, fixed_expert, y, s);
    case T_F16: return launch_down_t<T_F16>(b, act, ids, n_assign, fixed_expert, y, s);
    case T_BF16: return launch_down_t<T_BF16>(b, act, ids, n_assign, fixed_expert, y, s);
    case T_Q8_0: return launch_down_t<T_Q8_0>(b, act, ids, n_assign, fixed_expert, y, s);
    case T_Q4_K: return launch_down_t<T_Q4_K>(b, act, ids, n_assign, fixed_expert, y, s);
    default: return hipErrorInvalidValue;
    }
}

// ------------------------------------------------------------------------------------------
// combine: out[t] = (residual[t] +) sum over the token's slots in ascending expert id of
// w * y, multiply and add rounded separately.
// ------------------------------------------------------------------------------------------
constexpr int kCombineMaxK = 512;

__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y, const int32_t *__restrict__ ids,
                                                      const float *__restrict__ weights, int k, int hidden,
                                                      const float *__restrict__ residual, float *__restrict__ out) {
    __shared__ int s_order[kCombineMaxK];
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
    for (int s = threadIdx.x; s < k; s += blockDim.x) s_w[s] = weights[(size_t)t * k + s_order[s]];
    __syncthreads();
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < hidden; c += gridDim.y * blockDim.x) {
        float sum = 0.0f;
        for (int r = 0; r < k; r++) {
            const float v = y[((size_t)t * k + s_order[r]) * (size_t)hidden + c];
            sum = __fadd_rn(sum, __fmul_rn(s_w[r], v));
        }
        out[(size_t)t * hidden + c] = residual ? __fadd_rn(residual[(size_t)t * hidden + c], sum) : sum;
    }
}

hipError_t launch_combine(const float *y, const int32_t *ids, const float *weights, int n, int k, int hidden,
                          const float *residual, float *out, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (k > kCombineMaxK) return hipErrorInvalidValue;
    int ysplit = (hidden + 255) / 256;
    if (n >= 64) ysplit = 1;  // plenty of workgroups already
    dim3 block(256), grid(n, ysplit);
    combine_kernel<<<grid, block, 0, s>>>(y, ids, weights, k, hidden, residual, out);
    return hipGetLastError();
}

}  // namespace mummu
