// Device pieces shared by the packed-GEMV kernels: how the lanes of a wave split a quantized
// weight row, the lane's share of a 16-bit activation row, and the integer dot of the two.
#pragma once

#include "device_utils.h"
#include "qact.h"

namespace mummu {

// ------------------------------------------------------------------------------------------
// Lane geometry of one quantized weight row split in 32-element "units".
// ------------------------------------------------------------------------------------------
struct RowSplit {
    int units;        // units per row (in_dim / 32)
    int group;        // lanes that share a row (power of two, <= 64)
    int group_log2;
    int rows_per_it;  // rows a wave handles per iteration = 64 / group
};

__host__ __device__ inline RowSplit row_split(int in_dim) {
    RowSplit r;
    r.units = in_dim / 32;
    int lg = 0;
    while ((1 << lg) < r.units && lg < 6) lg++;
    r.group_log2 = lg;
    r.group = 1 << lg;
    r.rows_per_it = 64 >> lg;
    return r;
}

// Start elements of the two 16-element halves unit u of a row covers.
template <int WT>
__device__ inline void unit_halves(int u, int &e0, int &e1) {
    if constexpr (WT == T_Q4_K || WT == T_Q5_K) {
        int sb = u >> 3, up = u & 7;
        e0 = sb * 256 + (up >> 1) * 64 + (up & 1) * 16;  // low nibbles: elements of sub-block 2c
        e1 = e0 + 32;                                    // high nibbles: sub-block 2c+1
    } else if constexpr (WT == T_Q6_K) {
        // unit = 16 bytes of ql: their low nibbles are 16 consecutive elements, their high
        // nibbles the 16 elements 64 further on (ql byte offset inside the super-block = 16*up)
        int sb = u >> 3, up = u & 7;
        e0 = sb * 256 + (up >> 2) * 128 + (up & 3) * 16;
        e1 = e0 + 64;
    } else {
        e0 = u * 32;
        e1 = e0 + 16;
    }
}

// The lane's share of a quantized activation row: 32 values (two 16-element blocks).
template <int UPL>
struct LaneAct {
    int xh[UPL][8];   // hi bytes, 4 per word: words 0-3 first half, 4-7 second half
    int xl[UPL][8];   // lo bytes
    float s[UPL][2];    // scale of each half
    int sx[UPL][2];     // sum(xq) of each half
    float fsx[UPL][2];  // scale * sum(xq) of each half (what a block offset multiplies)
};

template <int WT, int UPL>
__device__ inline void load_lane_act(const QAct &q, size_t row, int d, int unit0, int units, LaneAct<UPL> &a) {
    const int8_t *hi = q.hi + row * (size_t)d;
    const int8_t *lo = q.lo + row * (size_t)d;
    const float *sc = q.scale + row * (size_t)(d / 16);
    const int32_t *sm = q.sum + row * (size_t)(d / 16);
#pragma unroll
    for (int i = 0; i < UPL; i++) {
        const int u = unit0 + 64 * i;
        const bool on = u < units;
        int e0, e1;
        unit_halves<WT>(on ? u : 0, e0, e1);
        const int4 h0 = *(const int4 *)(hi + e0), h1 = *(const int4 *)(hi + e1);
        const int4 l0 = *(const int4 *)(lo + e0), l1 = *(const int4 *)(lo + e1);
        a.xh[i][0] = h0.x; a.xh[i][1] = h0.y; a.xh[i][2] = h0.z; a.xh[i][3] = h0.w;
        a.xh[i][4] = h1.x; a.xh[i][5] = h1.y; a.xh[i][6] = h1.z; a.xh[i][7] = h1.w;
        a.xl[i][0] = l0.x; a.xl[i][1] = l0.y; a.xl[i][2] = l0.z; a.xl[i][3] = l0.w;
        a.xl[i][4] = l1.x; a.xl[i][5] = l1.y; a.xl[i][6] = l1.z; a.xl[i][7] = l1.w;
        // loaded whatever `on` says (the addresses are valid either way) and zeroed afterwards: a load
        // under a condition becomes a branch with a full wait in front of the loads that follow it
        const float s0 = sc[e0 >> 4], s1 = sc[e1 >> 4];
        const int x0 = sm[e0 >> 4], x1 = sm[e1 >> 4];
        a.s[i][0] = on ? s0 : 0.0f;
        a.s[i][1] = on ? s1 : 0.0f;
        a.sx[i][0] = on ? x0 : 0;
        a.sx[i][1] = on ? x1 : 0;
        a.fsx[i][0] = __fmul_rn(a.s[i][0], (float)a.sx[i][0]);
        a.fsx[i][1] = __fmul_rn(a.s[i][1], (float)a.sx[i][1]);
    }
}

// The lane's raw share of one quantized weight row, as loaded (nothing decoded yet).
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

// Legacy 32-element blocks (Q4_0 18 B, Q4_1 20 B, Q5_0 22 B, Q5_1 24 B): f16 d (, f16 m)
// (, u32 fifth bits), 16 bytes of nibbles.
template <int WT, int UPL>
struct RawLegacy {
    uint32_t dm[UPL];    // f16 d in the low half, f16 m in the high half (0 where the type has none)
    uint32_t qh[UPL];    // fifth bits (Q5_0, Q5_1)
    uint32_t q[UPL][4];  // nibbles
};
template <int UPL> struct RawRow<T_Q4_0, UPL> : RawLegacy<T_Q4_0, UPL> {};
template <int UPL> struct RawRow<T_Q4_1, UPL> : RawLegacy<T_Q4_1, UPL> {};
template <int UPL> struct RawRow<T_Q5_0, UPL> : RawLegacy<T_Q5_0, UPL> {};
template <int UPL> struct RawRow<T_Q5_1, UPL> : RawLegacy<T_Q5_1, UPL> {};
template <int UPL>
struct RawRow<T_Q5_K, UPL> {
    uint4 hdr[UPL];  // f16 d, f16 dmin, 12 B of 6-bit scales/mins
    uint4 qh[UPL];   // fifth bits of the lane's 16 byte positions (all four chunks)
    uint4 q[UPL];    // the lane's 16 bytes of nibbles
};
template <int UPL>
struct RawRow<T_Q6_K, UPL> {
    uint32_t ql[UPL][4];  // 16 bytes of low 4 bits
    uint32_t qh[UPL][4];  // the 16 bytes of high 2 bits they share with the unit 32 elements on
    uint32_t sc[UPL];     // int8 scale of the low-nibble elements | int8 scale of the high-nibble ones << 8
    uint32_t d[UPL];      // f16 super-block scale bits
};

constexpr bool is_legacy32(int t) { return t == T_Q4_0 || t == T_Q4_1 || t == T_Q5_0 || t == T_Q5_1; }

// An index every lane of the wave holds the same value of, told to the compiler (a value read from LDS or passed
// between lanes is uniform in fact, not by construction): addresses made of it and of kernel arguments stay in
// scalar registers.
__device__ __forceinline__ int uniform_index(int v) { return __builtin_amdgcn_readfirstlane(v); }

// The lane's share of the weight row that starts row_off bytes into the matrix at `base` (the same pointer in every
// lane - see uniform_index - so that a load is a scalar base plus a 32-bit lane offset: the matrix of one expert stays
// below 4 GB).
template <int WT, int UPL>
__device__ inline void load_row(const uint8_t *base, uint32_t row_off, int unit0, int units, bool ok, RawRow<WT, UPL> &r) {
    // Every lane loads unconditionally (a lane without a unit re-reads the row's last unit, a
    // lane of a row past the matrix reads the valid row the caller passes instead): straight-line
    // loads keep the wait counts exact, so rows still in flight are not waited for early.  What
    // must not count gets a zero block scale, which makes its contribution exactly 0.
#pragma unroll
    for (int i = 0; i < UPL; i++) {
        const int u = unit0 + 64 * i;
        const bool on = ok && u < units;
        const int uc = u < units ? u : units - 1;
        if constexpr (WT == T_Q4_K) {
            const uint8_t *blk = base + (row_off + (uint32_t)(uc >> 3) * 144u);
            r.hdr[i] = *(const uint4 *)blk;
            r.q[i] = *(const uint4 *)(blk + 16 + (uc & 7) * 16);
            r.hdr[i].x = on ? r.hdr[i].x : 0u;  // d = dmin = 0
        } else if constexpr (WT == T_Q5_K) {
            const uint8_t *blk = base + (row_off + (uint32_t)(uc >> 3) * 176u);  // 176 = 11 * 16: every piece is 16-byte aligned
            r.hdr[i] = *(const uint4 *)blk;
            r.qh[i] = *(const uint4 *)(blk + 16 + (uc & 1) * 16);
            r.q[i] = *(const uint4 *)(blk + 48 + (uc & 7) * 16);
            r.hdr[i].x = on ? r.hdr[i].x : 0u;
        } else if constexpr (WT == T_Q6_K) {
            const uint8_t *blk = base + (row_off + (uint32_t)(uc >> 3) * 210u);  // 2-byte aligned only
            const int up = uc & 7;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                __builtin_memcpy(&r.ql[i][w], blk + 16 * up + 4 * w, 4);
                __builtin_memcpy(&r.qh[i][w], blk + 128 + (up >> 2) * 32 + (up & 1) * 16 + 4 * w, 4);
            }
            const uint8_t *sc = blk + 192 + (up >> 2) * 8 + ((up >> 1) & 1) * 2 + (up & 1);
            r.sc[i] = (uint32_t)sc[0] | ((uint32_t)sc[4] << 8);
            uint16_t db;
            __builtin_memcpy(&db, blk + 208, 2);
            r.d[i] = on ? (uint32_t)db : 0u;
        } else if constexpr (is_legacy32(WT)) {
            constexpr bool has_m = WT == T_Q4_1 || WT == T_Q5_1;
            constexpr bool has_h = WT == T_Q5_0 || WT == T_Q5_1;
            const uint8_t *blk = base + (row_off + (uint32_t)uc * (uint32_t)block_bytes(WT));
            uint16_t db, mb = 0;
            __builtin_memcpy(&db, blk, 2);
            if constexpr (has_m) __builtin_memcpy(&mb, blk + 2, 2);
            r.dm[i] = on ? ((uint32_t)db | ((uint32_t)mb << 16)) : 0u;
            const uint8_t *p = blk + (has_m ? 4 : 2);
            r.qh[i] = 0u;
            if constexpr (has_h) {
                __builtin_memcpy(&r.qh[i], p, 4);
                p += 4;
            }
#pragma unroll
            for (int w = 0; w < 4; w++) __builtin_memcpy(&r.q[i][w], p + 4 * w, 4);
        } else {
            const uint8_t *blk = base + (row_off + (uint32_t)uc * 34u);
            uint16_t db;
            __builtin_memcpy(&db, blk, 2);
            r.d[i] = on ? (uint32_t)db : 0u;
#pragma unroll
            for (int w = 0; w < 8; w++) __builtin_memcpy(&r.q[i][w], blk + 2 + 4 * w, 4);  // 2-byte aligned
        }
    }
}

// The 6-bit (scale, min) of sub-blocks 2c and 2c+1 of a Q4_K / Q5_K super-block (ggml
// get_scale_min_k4), each pair packed as two bytes (sub-block 2c in byte 0), without a branch:
// y, z, w are the three words of the 12 scale bytes.
__device__ inline void k4_scale_min_pair(uint32_t y, uint32_t z, uint32_t w, int c, uint32_t &sc, uint32_t &mn) {
    const int sh = 16 * (c & 1);
    const uint32_t a = y >> sh, b = z >> sh, p = w >> sh;
    const uint32_t lo_sc = a & 0x3F3Fu, lo_mn = b & 0x3F3Fu;                   // sub-blocks 0..3: bytes j and j+4
    const uint32_t hi_sc = (p & 0x0F0Fu) | ((a >> 2) & 0x3030u);              // sub-blocks 4..7: low nibble of byte j+4,
    const uint32_t hi_mn = ((p >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);       // top two bits of byte j-4 (scale) / j (min)
    sc = c < 2 ? lo_sc : hi_sc;
    mn = c < 2 ? lo_mn : hi_mn;
}

// a . b over four signed bytes with nothing to add to: the first link of an accumulation chain.  (Written out for the
// first word of each chain below: with the chains started from variables that hold 0 the same unrolled loop compiles
// to a schedule that measures 7 % slower at four tokens per step.)
__device__ __forceinline__ int sdot4_first(int a, int b) { return __builtin_amdgcn_sdot4(a, b, 0, false); }

// The lane's partial of <row, activation> (formulas in the file comment).  A lane that loaded
// nothing holds zero scales and contributes exactly 0.
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
            // 6-bit (scale, min) of sub-blocks 2c, 2c+1, c fixed per lane
            uint32_t scp, mnp;
            k4_scale_min_pair(hdr.y, hdr.z, hdr.w, (u & 7) >> 1, scp, mnp);
            const float sc0 = (float)(scp & 0xFFu), sc1 = (float)((scp >> 8) & 0xFFu);
            const float mn0 = (float)(mnp & 0xFFu), mn1 = (float)((mnp >> 8) & 0xFFu);
            const uint32_t q[4] = {r.q[i].x, r.q[i].y, r.q[i].z, r.q[i].w};
            int lh = 0, ll = 0, hh = 0, hl = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                int lo = (int)(q[w] & 0x0F0F0F0Fu);
                int hi = (int)((q[w] >> 4) & 0x0F0F0F0Fu);
                if (w == 0) {
                    lh = sdot4_first(lo, a.xh[i][0]);
                    ll = sdot4_first(lo, a.xl[i][0]);
                    hh = sdot4_first(hi, a.xh[i][4]);
                    hl = sdot4_first(hi, a.xl[i][4]);
                    continue;
                }
                lh = __builtin_amdgcn_sdot4(lo, a.xh[i][w], lh, false);
                ll = __builtin_amdgcn_sdot4(lo, a.xl[i][w], ll, false);
                hh = __builtin_amdgcn_sdot4(hi, a.xh[i][4 + w], hh, false);
                hl = __builtin_amdgcn_sdot4(hi, a.xl[i][4 + w], hl, false);
            }
            // |sum(q*xq)| <= 15*32512*16 < 2^23: exact in f32
            const float p0 = (float)(lh * 256 + ll), p1 = (float)(hh * 256 + hl);
            const float pos = __builtin_fmaf(__fmul_rn(a.s[i][1], sc1), p1, __fmul_rn(__fmul_rn(a.s[i][0], sc0), p0));
            const float neg = __builtin_fmaf(a.fsx[i][1], mn1, __fmul_rn(a.fsx[i][0], mn0));
            acc = __builtin_fmaf(d, pos, acc);
            acc = __builtin_fmaf(-dmin, neg, acc);
        } else if constexpr (WT != T_Q8_0) {
            // Every other type: the two 16-element halves as non-negative byte codes c0, c1 with
            //     weight = A_h * code + B_h,
            // so the half's share is s_h * (A_h * sum(code * xq) + B_h * sum(xq)).
            uint32_t c0[4], c1[4];
            float A0, A1, B0, B1;
            if constexpr (is_legacy32(WT)) {
                const float d = half_bits_to_float((uint16_t)(r.dm[i] & 0xFFFFu));
                const float m = half_bits_to_float((uint16_t)(r.dm[i] >> 16));
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    c0[w] = r.q[i][w] & 0x0F0F0F0Fu;
                    c1[w] = (r.q[i][w] >> 4) & 0x0F0F0F0Fu;
                    if constexpr (WT == T_Q5_0 || WT == T_Q5_1) {
                        // fifth bit of element j is bit j of qh: 4 bits -> bit 4 of 4 bytes
                        c0[w] |= (((r.qh[i] >> (4 * w)) & 0xFu) * 0x02040810u) & 0x10101010u;
                        c1[w] |= (((r.qh[i] >> (16 + 4 * w)) & 0xFu) * 0x02040810u) & 0x10101010u;
                    }
                }
                A0 = A1 = d;
                B0 = B1 = WT == T_Q4_0 ? __fmul_rn(-8.0f, d) : (WT == T_Q5_0 ? __fmul_rn(-16.0f, d) : m);
            } else if constexpr (WT == T_Q5_K) {
                const int u = unit0 + 64 * i;
                const uint4 hdr = r.hdr[i];
                const float d = half_bits_to_float((uint16_t)(hdr.x & 0xFFFFu));
                const float dmin = half_bits_to_float((uint16_t)(hdr.x >> 16));
                const int c = (u & 7) >> 1;
                uint32_t scp, mnp;
                k4_scale_min_pair(hdr.y, hdr.z, hdr.w, c, scp, mnp);
                const float sc0 = (float)(scp & 0xFFu), sc1 = (float)((scp >> 8) & 0xFFu);
                const float mn0 = (float)(mnp & 0xFFu), mn1 = (float)((mnp >> 8) & 0xFFu);
                const uint32_t q[4] = {r.q[i].x, r.q[i].y, r.q[i].z, r.q[i].w};
                const uint32_t h[4] = {r.qh[i].x, r.qh[i].y, r.qh[i].z, r.qh[i].w};
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    c0[w] = (q[w] & 0x0F0F0F0Fu) | (((h[w] >> (2 * c)) & 0x01010101u) << 4);
                    c1[w] = ((q[w] >> 4) & 0x0F0F0F0Fu) | (((h[w] >> (2 * c + 1)) & 0x01010101u) << 4);
                }
                A0 = __fmul_rn(d, sc0);
                A1 = __fmul_rn(d, sc1);
                B0 = -__fmul_rn(dmin, mn0);
                B1 = -__fmul_rn(dmin, mn1);
            } else {  // Q6_K
                const int u = unit0 + 64 * i;
                const int jj = ((u & 7) >> 1) & 1;  // which pair of 2-bit fields of qh: (0, 4) or (2, 6)
                const float d = half_bits_to_float((uint16_t)r.d[i]);
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    c0[w] = (r.ql[i][w] & 0x0F0F0F0Fu) | (((r.qh[i][w] >> (2 * jj)) & 0x03030303u) << 4);
                    c1[w] = ((r.ql[i][w] >> 4) & 0x0F0F0F0Fu) | (((r.qh[i][w] >> (2 * jj + 4)) & 0x03030303u) << 4);
                }
                A0 = __fmul_rn(d, (float)(int)(int8_t)(r.sc[i] & 0xFFu));
                A1 = __fmul_rn(d, (float)(int)(int8_t)((r.sc[i] >> 8) & 0xFFu));
                B0 = __fmul_rn(-32.0f, A0);
                B1 = __fmul_rn(-32.0f, A1);
            }
            int h0 = 0, l0 = 0, h1 = 0, l1 = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                if (w == 0) {
                    h0 = sdot4_first((int)c0[0], a.xh[i][0]);
                    l0 = sdot4_first((int)c0[0], a.xl[i][0]);
                    h1 = sdot4_first((int)c1[0], a.xh[i][4]);
                    l1 = sdot4_first((int)c1[0], a.xl[i][4]);
                    continue;
                }
                h0 = __builtin_amdgcn_sdot4((int)c0[w], a.xh[i][w], h0, false);
                l0 = __builtin_amdgcn_sdot4((int)c0[w], a.xl[i][w], l0, false);
                h1 = __builtin_amdgcn_sdot4((int)c1[w], a.xh[i][4 + w], h1, false);
                l1 = __builtin_amdgcn_sdot4((int)c1[w], a.xl[i][4 + w], l1, false);
            }
            // codes <= 63 and |xq| <= 32512: every integer sum fits 32 bits
            acc = __builtin_fmaf(__fmul_rn(a.s[i][0], A0), (float)(h0 * 256 + l0), acc);
            acc = __builtin_fmaf(__fmul_rn(a.s[i][1], A1), (float)(h1 * 256 + l1), acc);
            acc = __builtin_fmaf(a.fsx[i][0], B0, acc);
            acc = __builtin_fmaf(a.fsx[i][1], B1, acc);
        } else {  // Q8_0
            const float d = half_bits_to_float((uint16_t)r.d[i]);
            int h0 = 0, l0 = 0, h1 = 0, l1 = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                if (w == 0) {
                    h0 = sdot4_first((int)r.q[i][0], a.xh[i][0]);
                    l0 = sdot4_first((int)r.q[i][0], a.xl[i][0]);
                    h1 = sdot4_first((int)r.q[i][4], a.xh[i][4]);
                    l1 = sdot4_first((int)r.q[i][4], a.xl[i][4]);
                    continue;
                }
                h0 = __builtin_amdgcn_sdot4((int)r.q[i][w], a.xh[i][w], h0, false);
                l0 = __builtin_amdgcn_sdot4((int)r.q[i][w], a.xl[i][w], l0, false);
                h1 = __builtin_amdgcn_sdot4((int)r.q[i][4 + w], a.xh[i][4 + w], h1, false);
                l1 = __builtin_amdgcn_sdot4((int)r.q[i][4 + w], a.xl[i][4 + w], l1, false);
            }
            const float t = __builtin_fmaf(a.s[i][0], (float)(h0 * 256 + l0), __fmul_rn(a.s[i][1], (float)(h1 * 256 + l1)));
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

// The same for NR rows at once against one activation row: the loads of all rows of an iteration
// go out together and every row has its own accumulator chain (a single row at a time leaves a
// wave waiting on one load and one chain of dependent fmas).  VEC = 8 only for the 16-bit types.
template <int WT, int VEC, int NR>
__device__ inline void rows_partial_f(const uint8_t *const (&rowp)[NR], const float *__restrict__ xrow, int in_dim, int lane,
                                      float (&acc)[NR]) {
    static_assert(VEC == 1 || VEC == 4 || (VEC == 8 && WT != T_F32), "vector widths: 1, 4, or 8 halfs");
#pragma unroll
    for (int r = 0; r < NR; r++) acc[r] = 0.0f;
    for (int i = lane * VEC; i < in_dim; i += 64 * VEC) {
        float xv[VEC];
        if constexpr (VEC == 1) {
            xv[0] = xrow[i];
        } else {
#pragma unroll
            for (int q = 0; q < VEC / 4; q++) {
                const float4 v = *(const float4 *)(xrow + i + 4 * q);
                xv[4 * q] = v.x; xv[4 * q + 1] = v.y; xv[4 * q + 2] = v.z; xv[4 * q + 3] = v.w;
            }
        }
        float w[NR][VEC];
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if constexpr (WT == T_F32) {
                if constexpr (VEC == 4) {
                    const float4 v = *(const float4 *)(rowp[r] + (size_t)i * 4);
                    w[r][0] = v.x; w[r][1] = v.y; w[r][2] = v.z; w[r][3] = v.w;
                } else {
                    w[r][0] = *(const float *)(rowp[r] + (size_t)i * 4);
                }
            } else {
                uint32_t raw[VEC >= 2 ? VEC / 2 : 1];
                if constexpr (VEC == 8) {
                    const uint4 v = *(const uint4 *)(rowp[r] + (size_t)i * 2);
                    raw[0] = v.x; raw[1] = v.y; raw[2] = v.z; raw[3] = v.w;
                } else if constexpr (VEC == 4) {
                    const uint2 v = *(const uint2 *)(rowp[r] + (size_t)i * 2);
                    raw[0] = v.x; raw[1] = v.y;
                } else {
                    raw[0] = *(const uint16_t *)(rowp[r] + (size_t)i * 2);
                }
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    const uint16_t h = (uint16_t)((raw[j / 2] >> (16 * (j & 1))) & 0xFFFFu);
                    w[r][j] = WT == T_F16 ? half_bits_to_float(h) : bf16_bits_to_float(h);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < NR; r++)
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[r] = __builtin_fmaf(w[r][j], xv[j], acc[r]);
    }
}

__host__ __device__ inline size_t type_row_bytes(int type, int in_dim) {
    return (size_t)(in_dim / block_elems(type)) * (size_t)block_bytes(type);
}

}  // namespace mummu
