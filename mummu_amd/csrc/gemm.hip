// SwiGLU expert products for batches (prefill): grouped GEMMs over the dispatch-sorted
// assignments on the matrix cores, one launch per projection for every routed expert of the
// layer.
//
// Reference semantics: per hit expert, y = down(silu(gate.x_e) * (up.x_e)) over the rows routed
// to it (nn/moe.rs:312-316, models/qwen4exp/experts.rs:1126-1135).
//
// Work list: (expert, first sorted position, rows <= 32*MT) tiles from the dispatch kernel;
// blockIdx.x walks that list (ragged and skewed expert loads just make it longer or shorter),
// blockIdx.y the output rows in slabs of 128.  A workgroup of 4 waves keeps a [32*MT x 64]
// activation tile and a [128 x 64] weight tile (two for gate+up) in LDS per K step; wave w owns
// output columns 32w..32w+31.  Weights are read from HBM once per tile in their GGUF bytes; the
// next K step's global loads are in flight while the current one is multiplied.
//
// Two arithmetic families:
//   F16 banks        v_mfma_f32_32x32x16_f16 on the stored halfs; activations rounded to f16.
//   Q8_0/Q4_K banks  v_mfma_i32_32x32x32_i8 on the stored integers (Q4_K nibbles widened to
//                    bytes) against activations quantized to 16 bits in two byte planes
//                    (x ~ s*(256*hi + lo), one scale per 64 elements): per 32-element block the
//                    integer sums are exact, C = 256*C_hi + C_lo, and the f32 accumulator takes
//                    s * sum_blocks(d_block * C).  Q4_K's offset term -dmin*m*sum(x) is one
//                    v_mfma_f32_32x32x2_f32 per K step over the per-block activation sums.
#include <cmath>
#include <type_traits>

#include "device_utils.h"
#include "kernels.h"

MUMMU_TRACE_UNIT(gemm)

namespace mummu {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int16v __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // staging registers: first-class vectors stay in VGPRs
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

constexpr int kBN = 128;            // output rows per workgroup
constexpr int kBK = 64;             // K step
constexpr int kLds = kBK + 8;       // f16 LDS row (halfs): 144 B keeps 16-byte reads conflict-free
constexpr int kLdsC = kBN + 4;      // f32 staging row of the gate/up epilogue

__device__ inline uint32_t pack_half2(float a, float b) {
    _Float16 h[2] = {(_Float16)a, (_Float16)b};
    uint32_t u;
    __builtin_memcpy(&u, h, 4);
    return u;
}

__host__ __device__ inline size_t gemm_row_bytes(int type, int in_dim) {
    return (size_t)(in_dim / block_elems(type)) * (size_t)block_bytes(type);
}

// Two biased halfs 1024 + byte from bytes 0, 1 (or 2, 3) of t.
__device__ inline half2v biased_pair(uint32_t t, bool upper) {
    const uint32_t u = __builtin_amdgcn_perm(0x64646464u, t, upper ? 0x04030402u : 0x04010400u);
    half2v h;
    __builtin_memcpy(&h, &u, 4);
    return h;
}

// Eight Q8_0 codes (two words of int8) times the block scale d as two halfs each, hi = rn(d * code) and
// lo = d * code - hi (exact: a 19-bit product, subnormal halfs included, which the vector and the matrix units
// both keep): a code b becomes the half 1024 + (b ^ 0x80) = b + 1152 by a byte permute, minus 1152 is exact.
__device__ inline void q8_half_planes(uint32_t c0, uint32_t c1, _Float16 d, half8 &hi, half8 &lo) {
    const half2v d2 = {d, d}, bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const uint32_t u0 = c0 ^ 0x80808080u, u1 = c1 ^ 0x80808080u;
    const half2v q[4] = {biased_pair(u0, false) - bias, biased_pair(u0, true) - bias, biased_pair(u1, false) - bias,
                         biased_pair(u1, true) - bias};
    half2v h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        h[j] = q[j] * d2;
        l[j] = __builtin_elementwise_fma(q[j], d2, -h[j]);
    }
    __builtin_memcpy(&hi, h, 16);
    __builtin_memcpy(&lo, l, 16);
}

// Epilogue shared by both families: acc register r of lane l is element
// (row 8*(r/4) + 4*(l/32) + r%4, column l%32) of the wave's 32x32 tile.
__device__ inline int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// Work-list entry (tile, output slab) of this workgroup of a 1-D grid.  Workgroups are dealt to
// the 8 XCDs round-robin by their linear id, each XCD with its own L2.  XCD j gets the contiguous
// run of tiles [j*ceil(T/8), (j+1)*ceil(T/8)) and walks it tile by tile with the slab index
// running fastest, so the workgroups resident on an XCD at any time are a few neighbouring tiles
// (the same expert, mostly) times all output slabs: the slabs of a tile share its activation rows
// in that L2 and the tiles of an expert share its weight slabs, instead of every L2 streaming
// everything.
__device__ inline bool xcd_tile(const int32_t *__restrict__ n_tiles, int slabs, int &tile, int &slab) {
    const int total = *n_tiles;
    const int per_xcd = (total + 7) >> 3;
    const int xcd = (int)(blockIdx.x & 7), i = (int)(blockIdx.x >> 3);
    slab = i % slabs;
    const int local = i / slabs;
    tile = xcd * per_xcd + local;
    return local < per_xcd && tile < total;
}

// ---------------------------------------------------------------------------------------
// F16 banks
// ---------------------------------------------------------------------------------------

// GATE_UP: A = x rounded to f16 (one small launch before this one: every output slab of a tile gathers the
//          tile's rows again, and as halfs that is half the traffic), rows gathered by token through `sorted`;
//          two weight matrices, epilogue act16[pos, n] = f16(silu(g) * u).
// else   : A = act16 (f16, rows already in sorted order), one matrix, y[pos, n] = f32 sum.
// BF16: the banks hold bf16; every weight becomes a half on its way into LDS (exact from 2^-14 up:
// a bf16 has 8 significant bits; smaller weights keep an absolute error below 2^-25).
// WT = T_Q8_0: the banks hold Q8_0 blocks (34 bytes: f16 d, 32 int8 codes).  A thread's share of a row and K step is
// then 8 codes and their block's d; the codes go to LDS as they are, and the wave that owns a column turns its 8
// codes of an instruction into two operands, hi + lo = d * code exactly, and multiplies both: twice the matrix
// work of an f16 bank at half the bytes, and the weights lose nothing (x and the activations between the two
// products are halfs, as for every bank of this kernel).  Needs |d| * 128 inside the half range.
template <bool GATE_UP, int MT, int WT>
__global__ __launch_bounds__(256) void grouped_gemm_f16_kernel(
    const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, const _Float16 *__restrict__ act_in,
    const int32_t *__restrict__ sorted, int k_slots, const int32_t *__restrict__ tiles, const int32_t *__restrict__ n_tiles,
    int in_dim, int out_dim, _Float16 *__restrict__ act_out, float *__restrict__ y_out) {
    constexpr int NB = GATE_UP ? 2 : 1;
    constexpr int BM = 32 * MT;
    constexpr bool BF16 = WT == T_BF16, Q8 = WT == T_Q8_0;
    constexpr int kQRow = kBK + 8;   // a row of codes in LDS (bytes): 72 keeps the 8-byte reads of 32 columns conflict-free
    __shared__ __attribute__((aligned(16))) _Float16 s_a[BM][kLds];
    __shared__ __attribute__((aligned(16))) _Float16 s_b[Q8 ? 1 : NB][Q8 ? 1 : kBN][kLds];
    __shared__ __attribute__((aligned(16))) uint8_t s_q[Q8 ? NB : 1][Q8 ? kBN : 1][kQRow];   // Q8_0: the step's codes ...
    __shared__ _Float16 s_d[Q8 ? NB : 1][Q8 ? kBN : 1][2];                                    // ... and the d of its two blocks

    int tile, slab;
    if (!xcd_tile(n_tiles, (out_dim + kBN - 1) / kBN, tile, slab)) return;
    const int e = tiles[3 * tile], p0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = slab * kBN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    static_assert(WT == T_F16 || WT == T_BF16 || WT == T_Q8_0, "banks this kernel reads");
    const size_t row_bytes = Q8 ? (size_t)(in_dim / 32) * 34 : (size_t)in_dim * 2;

    // weight tile: a K step of one row is 128 contiguous bytes = 8 lanes x 16 B, so one load
    // instruction of a wave covers 8 whole rows; thread -> chunk tid%8 of rows tid/8 + 32*i
    // (Q8_0: the step is two blocks = 68 bytes; chunk c = codes 8 (c % 4) .. +7 of block c / 4, at byte
    // 34 (c / 4) + 2 + 8 (c % 4) of the step)
    const int b_chunk = tid & 7;
    const size_t b_chunk_at = Q8 ? (size_t)(34 * (b_chunk >> 2) + 2 + 8 * (b_chunk & 3)) : (size_t)b_chunk * 16;
    const uint8_t *b_ptr[NB][4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (tid >> 3) + 32 * i;
        const int b_out = n0 + r < out_dim ? n0 + r : out_dim - 1;  // clamped; never stored
        b_ptr[0][i] = w0 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes + b_chunk_at;
        if (GATE_UP) b_ptr[NB - 1][i] = w1 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes + b_chunk_at;
    }

    // activation tile: 8 threads per row, 8 halfs each (MT passes of 32 rows)
    constexpr int A_PASSES = MT;
    const int a_col = (tid & 7) * 8;
    // rows past the tile's end read the tile's last row: their products are never stored
    const _Float16 *a_src16[A_PASSES];
    int a_row[A_PASSES];
#pragma unroll
    for (int p = 0; p < A_PASSES; p++) {
        a_row[p] = p * 32 + (tid >> 3);
        const int r = a_row[p] < rows ? a_row[p] : rows - 1;
        const int src = GATE_UP ? sorted[p0 + r] / k_slots : p0 + r;
        a_src16[p] = act_in + (size_t)src * (size_t)in_dim + a_col;
    }

    float16v acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[b][m][r] = 0.0f;

    u32x4 rb[NB][4];
    u32x4 ra16[A_PASSES];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (Q8) {
                    // 8 codes (2-byte aligned) and the d of their block, 2 + 8 (c % 4) bytes before them
                    const uint8_t *p = b_ptr[b][i] + (size_t)(k0 >> 5) * 34;
                    uint32_t c0, c1;
                    uint16_t db;
                    __builtin_memcpy(&c0, p, 4);
                    __builtin_memcpy(&c1, p + 4, 4);
                    __builtin_memcpy(&db, p - (2 + 8 * (b_chunk & 3)), 2);
                    rb[b][i] = u32x4{c0, c1, (uint32_t)db, 0u};
                } else {
                    rb[b][i] = *(const u32x4 *)(b_ptr[b][i] + (size_t)k0 * 2);
                }
            }
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) ra16[p] = *(const u32x4 *)(a_src16[p] + k0);
    };
    // The K loop starts at a slab-dependent step and wraps.  An f16 row of 2048 elements is 4096
    // bytes - the period of the memory channel interleave - so one K step of ALL rows lives in one
    // channel, and with every workgroup of the chip marching through K in lockstep the whole
    // launch would queue on one or two channels at a time.  Rotating by slab spreads the slabs
    // over the channels; a token's result still depends only on its output slab, never on which
    // tile or batch it arrived in.
    const int n_steps = in_dim / kBK;
    const int n_slabs = (out_dim + kBN - 1) / kBN;
    const int rot = (slab * (n_steps / n_slabs > 0 ? n_steps / n_slabs : 1)) % n_steps;
    auto step_k0 = [&](int step) { return ((step + rot) % n_steps) * kBK; };
    fetch(step_k0(0));

    MUMMU_TIMER_DECL;
    for (int step = 0; step < n_steps; step++) {
        MUMMU_TIMER_MARK(0);
        // registers -> LDS
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                u32x4 v = rb[b][i];
                if constexpr (Q8) {
                    *(uint2 *)&s_q[b][(tid >> 3) + 32 * i][b_chunk * 8] = make_uint2(v[0], v[1]);
                    if ((b_chunk & 3) == 0) {
                        const uint16_t db = (uint16_t)v[2];
                        __builtin_memcpy(&s_d[b][(tid >> 3) + 32 * i][b_chunk >> 2], &db, 2);
                    }
                    continue;
                }
                if (BF16) {
#pragma unroll
                    for (int q = 0; q < 4; q++) v[q] = pack_half2(__uint_as_float(v[q] << 16), __uint_as_float(v[q] & 0xFFFF0000u));
                }
                *(u32x4 *)&s_b[b][(tid >> 3) + 32 * i][b_chunk * 8] = v;
            }
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) *(u32x4 *)&s_a[a_row[p]][a_col] = ra16[p];
        MUMMU_TIMER_MARK(1);
        __syncthreads();
        MUMMU_TIMER_MARK(2);
        if (step + 1 < n_steps) fetch(step_k0(step + 1));
        MUMMU_TIMER_MARK(3);
        // multiply: wave owns columns 32*wave .. +31
#pragma unroll
        for (int kk = 0; kk < kBK / 16; kk++) {
            half8 bfrag[NB], bfrag_lo[NB];
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if constexpr (Q8) {
                    const uint2 c = *(const uint2 *)&s_q[b][32 * wave + (lane & 31)][kk * 16 + (lane >> 5) * 8];
                    q8_half_planes(c.x, c.y, s_d[b][32 * wave + (lane & 31)][kk >> 1], bfrag[b], bfrag_lo[b]);
                } else {
                    bfrag[b] = *(const half8 *)&s_b[b][32 * wave + (lane & 31)][kk * 16 + (lane >> 5) * 8];
                }
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const half8 afrag = *(const half8 *)&s_a[32 * m + (lane & 31)][kk * 16 + (lane >> 5) * 8];
#pragma unroll
                for (int b = 0; b < NB; b++) acc[b][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag[b], acc[b][m], 0, 0, 0);
                if constexpr (Q8) {
#pragma unroll
                    for (int b = 0; b < NB; b++)
                        acc[b][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag_lo[b], acc[b][m], 0, 0, 0);
                }
            }
        }
        MUMMU_TIMER_MARK(4);
        __syncthreads();
        MUMMU_TIMER_MARK(5);
    }
    MUMMU_TIMER_STORE;

    const int n = n0 + 32 * wave + (lane & 31);
    if (n < out_dim) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = 32 * m + acc_row(r, lane);
                if (row < rows) {
                    const size_t o = (size_t)(p0 + row) * (size_t)out_dim + (size_t)n;
                    if (GATE_UP) act_out[o] = (_Float16)__fmul_rn(det_silu(acc[0][m][r]), acc[NB - 1][m][r]);
                    else y_out[o] = acc[0][m][r];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// block-quantized banks (Q8_0, Q4_K, Q5_K, Q6_K, Q4_0, Q4_1, Q5_0, Q5_1)
// ---------------------------------------------------------------------------------------

// Raw bytes of one thread's share of a weight tile: one 32-element block of one row.
template <int WT>
struct RawQ;
template <>
struct RawQ<T_Q8_0> {
    uint32_t d;
    uint32_t q[8];
};
template <>
struct RawQ<T_Q4_K> {
    uint4 hdr;
    uint4 q[2];
};
template <>
struct RawQ<T_Q5_K> {
    uint4 hdr;
    uint4 qh[2];  // fifth bits of the 32 byte positions (all four chunks)
    uint4 q[2];
};
template <>
struct RawQ<T_Q6_K> {
    uint32_t ql[8];  // 32 bytes of low 4 bits (one nibble of each is this block's)
    uint32_t qh[8];  // 32 bytes of high 2 bits (one field of each is this block's)
    uint32_t sc;     // the block's two int8 scales (16 elements each)
    uint32_t d;
};
struct RawLegacyQ {
    uint32_t dm;  // f16 d | f16 m << 16
    uint32_t qh;  // fifth bits (Q5_0, Q5_1)
    uint32_t q[4];
};
template <> struct RawQ<T_Q4_0> : RawLegacyQ {};
template <> struct RawQ<T_Q4_1> : RawLegacyQ {};
template <> struct RawQ<T_Q5_0> : RawLegacyQ {};
template <> struct RawQ<T_Q5_1> : RawLegacyQ {};

constexpr bool gemm_legacy32(int t) { return t == T_Q4_0 || t == T_Q4_1 || t == T_Q5_0 || t == T_Q5_1; }
// weight = scale * code + offset with a non-zero offset (the offset term rides on an f32 MFMA)
constexpr bool gemm_has_offset(int t) { return t != T_Q8_0 && t != T_Q6_K; }
// one scale per 16 elements instead of per 32 (the integer products are split at 16)
constexpr bool gemm_sub16(int t) { return t == T_Q6_K; }

// rowp: start of the weight row; k0: first element of the K step (multiple of 64); half: which
// 32-element block of the step.
template <int WT>
__device__ inline void load_q(const uint8_t *__restrict__ rowp, int k0, int half, RawQ<WT> &r) {
    if constexpr (WT == T_Q8_0) {
        const uint8_t *blk = rowp + (size_t)(k0 / 32 + half) * 34;
        uint16_t db;
        __builtin_memcpy(&db, blk, 2);
        r.d = db;
#pragma unroll
        for (int w = 0; w < 8; w++) __builtin_memcpy(&r.q[w], blk + 2 + 4 * w, 4);
    } else if constexpr (WT == T_Q4_K) {
        const uint8_t *blk = rowp + (size_t)(k0 >> 8) * 144;
        r.hdr = *(const uint4 *)blk;
        const uint4 *q = (const uint4 *)(blk + 16 + ((k0 & 255) >> 6) * 32);
        r.q[0] = q[0];
        r.q[1] = q[1];
    } else if constexpr (WT == T_Q5_K) {
        const uint8_t *blk = rowp + (size_t)(k0 >> 8) * 176;
        r.hdr = *(const uint4 *)blk;
        r.qh[0] = *(const uint4 *)(blk + 16);
        r.qh[1] = *(const uint4 *)(blk + 32);
        const uint4 *q = (const uint4 *)(blk + 48 + ((k0 & 255) >> 6) * 32);
        r.q[0] = q[0];
        r.q[1] = q[1];
    } else if constexpr (WT == T_Q6_K) {
        const uint8_t *blk = rowp + (size_t)(k0 >> 8) * 210;  // 2-byte aligned only
        const int within = (k0 & 255) + 32 * half, n = within >> 7, j = (within & 127) >> 5;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            __builtin_memcpy(&r.ql[w], blk + 64 * n + 32 * (j & 1) + 4 * w, 4);
            __builtin_memcpy(&r.qh[w], blk + 128 + 32 * n + 4 * w, 4);
        }
        uint16_t sb, db;
        __builtin_memcpy(&sb, blk + 192 + 8 * n + 2 * j, 2);
        __builtin_memcpy(&db, blk + 208, 2);
        r.sc = sb;
        r.d = db;
    } else {
        constexpr bool has_m = WT == T_Q4_1 || WT == T_Q5_1;
        constexpr bool has_h = WT == T_Q5_0 || WT == T_Q5_1;
        const uint8_t *blk = rowp + (size_t)(k0 / 32 + half) * block_bytes(WT);
        uint16_t db, mb = 0;
        __builtin_memcpy(&db, blk, 2);
        if constexpr (has_m) __builtin_memcpy(&mb, blk + 2, 2);
        r.dm = (uint32_t)db | ((uint32_t)mb << 16);
        const uint8_t *p = blk + (has_m ? 4 : 2);
        r.qh = 0u;
        if constexpr (has_h) {
            __builtin_memcpy(&r.qh, p, 4);
            p += 4;
        }
#pragma unroll
        for (int w = 0; w < 4; w++) __builtin_memcpy(&r.q[w], p + 4 * w, 4);
    }
}

// ggml get_scale_min_k4 on the 12 scale bytes held in three words.
__device__ inline void k4_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, uint32_t &sc, uint32_t &mn) {
    auto byte_of = [&](int k) -> uint32_t {
        const uint32_t w = k < 4 ? s0 : (k < 8 ? s1 : s2);
        return (w >> (8 * (k & 3))) & 0xFFu;
    };
    if (j < 4) {
        sc = byte_of(j) & 63u;
        mn = byte_of(j + 4) & 63u;
    } else {
        const uint32_t hi = byte_of(j + 4);
        sc = (hi & 0x0Fu) | ((byte_of(j - 4) >> 6) << 4);
        mn = (hi >> 4) | ((byte_of(j) >> 6) << 4);
    }
}

// The same for sub-blocks 2c and 2c+1 at once, each pair packed as two bytes (sub-block 2c in byte 0),
// without a branch.
__device__ inline void k4_scale_min_both(uint32_t y, uint32_t z, uint32_t w, int c, uint32_t &sc, uint32_t &mn) {
    const int sh = 16 * (c & 1);
    const uint32_t a = y >> sh, b = z >> sh, p = w >> sh;
    const uint32_t lo_sc = a & 0x3F3Fu, lo_mn = b & 0x3F3Fu;
    const uint32_t hi_sc = (p & 0x0F0Fu) | ((a >> 2) & 0x3030u);
    const uint32_t hi_mn = ((p >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
    sc = c < 2 ? lo_sc : hi_sc;
    mn = c < 2 ? lo_mn : hi_mn;
}

// The block's 32 integers as bytes in element order, with weight = scale * byte + offset.
// Types with one scale per 16 elements return the second half's scale in scale1 (else scale1 =
// scale).  Bytes are codes 0..31 (unsigned) or, for Q8_0 / Q6_K, signed values.
template <int WT>
__device__ inline void expand_q(const RawQ<WT> &r, int k0, int half, uint32_t (&q)[8], float &scale, float &scale1,
                                float &offset) {
    if constexpr (WT == T_Q8_0) {
#pragma unroll
        for (int w = 0; w < 8; w++) q[w] = r.q[w];
        scale = scale1 = half_bits_to_float((uint16_t)r.d);
        offset = 0.0f;
    } else if constexpr (WT == T_Q4_K || WT == T_Q5_K) {
        const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFFu));
        const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
        const int c = (k0 & 255) >> 6;
        const int j = 2 * c + half;  // sub-block: low nibbles first, then high
        uint32_t sc, mn;
        k4_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, j, sc, mn);
        scale = scale1 = __fmul_rn(d, (float)sc);
        offset = -__fmul_rn(dmin, (float)mn);
        const uint32_t qw[8] = {r.q[0].x, r.q[0].y, r.q[0].z, r.q[0].w, r.q[1].x, r.q[1].y, r.q[1].z, r.q[1].w};
#pragma unroll
        for (int w = 0; w < 8; w++) q[w] = half ? (qw[w] >> 4) & 0x0F0F0F0Fu : qw[w] & 0x0F0F0F0Fu;
        if constexpr (WT == T_Q5_K) {
            const uint32_t hw[8] = {r.qh[0].x, r.qh[0].y, r.qh[0].z, r.qh[0].w, r.qh[1].x, r.qh[1].y, r.qh[1].z, r.qh[1].w};
#pragma unroll
            for (int w = 0; w < 8; w++) q[w] |= ((hw[w] >> j) & 0x01010101u) << 4;
        }
    } else if constexpr (WT == T_Q6_K) {
        const int within = (k0 & 255) + 32 * half, j = (within & 127) >> 5;
        const float d = half_bits_to_float((uint16_t)r.d);
        scale = __fmul_rn(d, (float)(int)(int8_t)(r.sc & 0xFFu));
        scale1 = __fmul_rn(d, (float)(int)(int8_t)((r.sc >> 8) & 0xFFu));
        offset = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t nib = j < 2 ? r.ql[w] & 0x0F0F0F0Fu : (r.ql[w] >> 4) & 0x0F0F0F0Fu;
            const uint32_t code = nib | (((r.qh[w] >> (2 * j)) & 0x03030303u) << 4);   // 0..63 per byte
            q[w] = ((code | 0x80808080u) - 0x20202020u) ^ 0x80808080u;                  // minus 32, byte-wise
        }
    } else {  // Q4_0, Q4_1, Q5_0, Q5_1
        const float d = half_bits_to_float((uint16_t)(r.dm & 0xFFFFu));
        const float m = half_bits_to_float((uint16_t)(r.dm >> 16));
#pragma unroll
        for (int w = 0; w < 4; w++) {
            q[w] = r.q[w] & 0x0F0F0F0Fu;
            q[4 + w] = (r.q[w] >> 4) & 0x0F0F0F0Fu;
            if constexpr (WT == T_Q5_0 || WT == T_Q5_1) {
                q[w] |= (((r.qh >> (4 * w)) & 0xFu) * 0x02040810u) & 0x10101010u;
                q[4 + w] |= (((r.qh >> (16 + 4 * w)) & 0xFu) * 0x02040810u) & 0x10101010u;
            }
        }
        scale = scale1 = d;
        offset = WT == T_Q4_0 ? __fmul_rn(-8.0f, d) : (WT == T_Q5_0 ? __fmul_rn(-16.0f, d) : m);
    }
}


// ---------------------------------------------------------------------------------------
// F32 banks: v_mfma_f32_32x32x2_f32, everything stays f32 (tolerance class 1e-5)
// ---------------------------------------------------------------------------------------
constexpr int kFK = 32;          // K step (floats): a row's step is 128 B = 8 lanes x 16 B, as for the halfs
constexpr int kLdsF = kFK + 4;   // LDS row (floats)

// Same tiles and work list as the f16 kernel.  One MFMA multiplies two K values: lane half g supplies
// k = 16 g + j of the step for j = 0..15, so a lane's operands for four consecutive instructions are
// one 16-byte LDS read.
// GATE_UP: A = x (gathered by token through `sorted`), two weight matrices, act_out[pos, n] = silu(g) * u.
// else   : A = the f32 activation rows in sorted order, one matrix, y[pos, n] = the sum.
template <bool GATE_UP, int MT>
__global__ __launch_bounds__(256) void grouped_gemm_f32_kernel(
    const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, const float *__restrict__ a_in,
    const int32_t *__restrict__ sorted, int k_slots, const int32_t *__restrict__ tiles, const int32_t *__restrict__ n_tiles,
    int in_dim, int out_dim, float *__restrict__ act_out, float *__restrict__ y_out) {
    constexpr int NB = GATE_UP ? 2 : 1;
    constexpr int BM = 32 * MT;
    __shared__ __attribute__((aligned(16))) float s_a[BM][kLdsF];
    __shared__ __attribute__((aligned(16))) float s_b[NB][kBN][kLdsF];

    int tile, slab;
    if (!xcd_tile(n_tiles, (out_dim + kBN - 1) / kBN, tile, slab)) return;
    const int e = tiles[3 * tile], p0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = slab * kBN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t row_bytes = (size_t)in_dim * 4;

    // weight tile: thread -> 16-byte chunk tid%8 of rows tid/8 + 32*i; activation tile alike, MT passes
    const int chunk = tid & 7;
    const uint8_t *b_ptr[NB][4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (tid >> 3) + 32 * i;
        const int b_out = n0 + r < out_dim ? n0 + r : out_dim - 1;  // clamped; never stored
        b_ptr[0][i] = w0 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes + (size_t)chunk * 16;
        if (GATE_UP) b_ptr[NB - 1][i] = w1 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes + (size_t)chunk * 16;
    }
    const float *a_src[MT];
#pragma unroll
    for (int p = 0; p < MT; p++) {
        // rows past the tile's end read the tile's last row: their products are never stored
        const int r = 32 * p + (tid >> 3) < rows ? 32 * p + (tid >> 3) : rows - 1;
        const int src = GATE_UP ? sorted[p0 + r] / k_slots : p0 + r;
        a_src[p] = a_in + (size_t)src * (size_t)in_dim + chunk * 4;
    }

    float16v acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[b][m][r] = 0.0f;

    f32x4 rb[NB][4], ra[MT];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int i = 0; i < 4; i++) rb[b][i] = *(const f32x4 *)(b_ptr[b][i] + (size_t)k0 * 4);
#pragma unroll
        for (int p = 0; p < MT; p++) ra[p] = *(const f32x4 *)(a_src[p] + k0);
    };
    fetch(0);
    const int col = 32 * wave + (lane & 31), g = lane >> 5;
    for (int k0 = 0; k0 < in_dim; k0 += kFK) {
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int i = 0; i < 4; i++) *(f32x4 *)&s_b[b][(tid >> 3) + 32 * i][chunk * 4] = rb[b][i];
#pragma unroll
        for (int p = 0; p < MT; p++) *(f32x4 *)&s_a[32 * p + (tid >> 3)][chunk * 4] = ra[p];
        __syncthreads();
        if (k0 + kFK < in_dim) fetch(k0 + kFK);
#pragma unroll
        for (int jq = 0; jq < 4; jq++) {
            f32x4 bv[NB];
#pragma unroll
            for (int b = 0; b < NB; b++) bv[b] = *(const f32x4 *)&s_b[b][col][16 * g + 4 * jq];
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const f32x4 av = *(const f32x4 *)&s_a[32 * m + (lane & 31)][16 * g + 4 * jq];
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int b = 0; b < NB; b++) acc[b][m] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[q], bv[b][q], acc[b][m], 0, 0, 0);
            }
        }
        __syncthreads();
    }

    const int n = n0 + col;
    if (n < out_dim) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = 32 * m + acc_row(r, lane);
                if (row < rows) {
                    const size_t o = (size_t)(p0 + row) * (size_t)out_dim + (size_t)n;
                    if (GATE_UP) act_out[o] = __fmul_rn(det_silu(acc[0][m][r]), acc[NB - 1][m][r]);
                    else y_out[o] = acc[0][m][r];
                }
            }
        }
    }
}

template <bool GATE_UP, int MT, int KS>
struct QTileLds {
    static constexpr int NB = GATE_UP ? 2 : 1;
    static constexpr int BM = 32 * MT;
    static constexpr int kRow = KS * kBK + 16;                // LDS row (bytes): 80 or 144 B keep 16-byte reads conflict-free
    static constexpr int kA = 2 * BM * kRow;                  // hi and lo planes
    static constexpr int kB = NB * kBN * kRow;
    static constexpr int kC = GATE_UP ? BM * kLdsC * 4 : 0;   // f32 staging of the epilogue (aliases A and B)
    static constexpr int kBytes = (kA + kB) > kC ? (kA + kB) : kC;
};

// GATE_UP: A = xq rows gathered by token through `sorted`; epilogue quantizes silu(g)*u into
//          act_out rows in sorted order.
// else   : A = act_in rows in sorted order; y[pos, n] = f32 sum.
// KS: 64-element K steps staged per barrier pair.  With KS = 2 (in_dim a multiple of 128) the two
// threads of a weight row each load and expand a whole step of their own instead of the two blocks
// of one step: the same registers keep twice the bytes in flight, which is what a launch that
// streams its weights with few rows per expert is short of; the arithmetic and its order per
// output element are the same.
template <int WT, bool GATE_UP, int MT, int KS>
__global__ __launch_bounds__(256, 2) void grouped_gemm_q_kernel(
    const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, QAct64 a_in, const int32_t *__restrict__ sorted,
    int k_slots, const int32_t *__restrict__ tiles, const int32_t *__restrict__ n_tiles, int in_dim, int out_dim,
    QAct64 act_out, float *__restrict__ y_out) {
    using L = QTileLds<GATE_UP, MT, KS>;
    constexpr int NB = L::NB, BM = L::BM, kRow = L::kRow;
    __shared__ __attribute__((aligned(16))) uint8_t s_raw[L::kBytes];
    __shared__ __attribute__((aligned(16))) float s_as[KS][BM];   // activation scale of each K step, per tile row
    __shared__ float s_am[BM][2 * KS];                            // activation ssum of their blocks
    constexpr bool OFFSET = gemm_has_offset(WT), SUB16 = gemm_sub16(WT);
    constexpr int NSC = SUB16 ? 4 : 2;
    __shared__ float s_bd[NB][kBN][NSC * KS];                     // weight scales of the K steps (per 32 or per 16 elements)
    __shared__ float s_bm[NB][kBN][2 * KS];                       // weight block offsets (types that have one)
    auto s_a = [&](int plane, int row) -> uint8_t * { return s_raw + ((size_t)plane * BM + row) * kRow; };
    auto s_b = [&](int b, int row) -> uint8_t * { return s_raw + L::kA + ((size_t)b * kBN + row) * kRow; };

    int tile, slab;
    if (!xcd_tile(n_tiles, (out_dim + kBN - 1) / kBN, tile, slab)) return;
    const int e = tiles[3 * tile], p0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = slab * kBN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t row_bytes = gemm_row_bytes(WT, in_dim);

    // weight tile: thread -> (row, block of the K step), or with two steps per stage (row, step)
    // and both blocks of that step
    const int b_row = tid >> 1, b_half = tid & 1;
    constexpr bool SHARED = WT == T_Q4_K || WT == T_Q5_K;  // one load holds both blocks of a step
    constexpr int NBLK = KS, NRAW = (KS == 2 && !SHARED) ? 2 : 1;
    const int b_out = n0 + b_row < out_dim ? n0 + b_row : out_dim - 1;  // clamped; never stored
    const uint8_t *b_ptr[NB];
    b_ptr[0] = w0 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes;
    if (GATE_UP) b_ptr[NB - 1] = w1 + ((size_t)e * (size_t)out_dim + (size_t)b_out) * row_bytes;

    // source row of tile row r (-1: past the tile's rows)
    auto source_row = [&](int r) -> int {
        if (r >= rows) return -1;
        return GATE_UP ? sorted[p0 + r] / k_slots : p0 + r;
    };
    // activation tile: thread -> (plane, row, 16-byte chunk), MT * KS passes of 32 / KS rows
    constexpr int A_PASSES = MT * KS, A_CHUNKS = 4 * KS, A_ROWS = 32 / KS;
    const int a_plane = tid >> 7, a_chunk = tid & (A_CHUNKS - 1);
    const int8_t *a_src[A_PASSES];
    int a_row[A_PASSES];
#pragma unroll
    for (int p = 0; p < A_PASSES; p++) {
        a_row[p] = A_ROWS * p + ((tid / A_CHUNKS) & (A_ROWS - 1));
        const int src = source_row(a_row[p]);
        a_src[p] = src < 0 ? nullptr : (a_plane ? a_in.lo : a_in.hi) + (size_t)src * (size_t)in_dim + a_chunk * 16;
    }
    // its scales: thread t < KS*BM -> scale of (row t % BM, step t / BM); thread t < 2*KS*BM -> ssum of
    // (row t / (2 KS), block t % (2 KS))
    const int src_s = tid < KS * BM ? source_row(tid % BM) : -1;
    const int src_m = tid < 2 * KS * BM ? source_row(tid / (2 * KS)) : -1;
    const float *as_ptr = src_s < 0 ? nullptr : a_in.scale + (size_t)src_s * (size_t)(in_dim / 64) + tid / BM;
    const float *am_ptr = src_m < 0 ? nullptr : a_in.ssum + (size_t)src_m * (size_t)(in_dim / 32) + (tid & (2 * KS - 1));

    float16v acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[b][m][r] = 0.0f;

    // raw registers of the next stage: refilled right after a stage has been expanded into LDS, so the loads fly
    // under the products.  (A second set, two stages ahead, was measured and bought nothing: with few rows per
    // expert the launch already moves 3.5 TB/s of 72-byte row pieces.)
    RawQ<WT> rb[NB][NRAW];
    uint4 ra[A_PASSES];
    float ras = 0.0f, ram = 0.0f;
    auto fetch = [&](int k0) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if constexpr (KS == 1) {
                load_q<WT>(b_ptr[b], k0, b_half, rb[b][0]);
            } else {
#pragma unroll
                for (int hf = 0; hf < NRAW; hf++) load_q<WT>(b_ptr[b], k0 + kBK * b_half, hf, rb[b][hf]);
            }
        }
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) ra[p] = a_src[p] ? *(const uint4 *)(a_src[p] + k0) : make_uint4(0, 0, 0, 0);
        ras = as_ptr ? as_ptr[k0 >> 6] : 0.0f;
        if (OFFSET) ram = am_ptr ? am_ptr[k0 >> 5] : 0.0f;
    };

    const int col = 32 * wave + (lane & 31), g = lane >> 5;
    MUMMU_TIMER_DECL;
    // registers of set S -> LDS
    auto stage = [&](int k0) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if constexpr (KS == 2 && SHARED) {
                // both blocks of this thread's step come out of one 32-byte chunk: header, scale pair and nibble
                // split are done once (same values, bit for bit, as two expand_q calls)
                const RawQ<WT> &r = rb[b][0];
                const int c = ((k0 + kBK * b_half) & 255) >> 6;
                const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFFu));
                const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
                uint32_t scp, mnp;
                k4_scale_min_both(r.hdr.y, r.hdr.z, r.hdr.w, c, scp, mnp);
                const uint32_t qw[8] = {r.q[0].x, r.q[0].y, r.q[0].z, r.q[0].w, r.q[1].x, r.q[1].y, r.q[1].z, r.q[1].w};
                uint32_t lo[8], hi[8];
#pragma unroll
                for (int w = 0; w < 8; w++) {
                    lo[w] = qw[w] & 0x0F0F0F0Fu;
                    hi[w] = (qw[w] >> 4) & 0x0F0F0F0Fu;
                }
                if constexpr (WT == T_Q5_K) {
                    const uint32_t hw[8] = {r.qh[0].x, r.qh[0].y, r.qh[0].z, r.qh[0].w, r.qh[1].x, r.qh[1].y, r.qh[1].z, r.qh[1].w};
#pragma unroll
                    for (int w = 0; w < 8; w++) {
                        lo[w] |= ((hw[w] >> (2 * c)) & 0x01010101u) << 4;
                        hi[w] |= ((hw[w] >> (2 * c + 1)) & 0x01010101u) << 4;
                    }
                }
                uint4 *dst = (uint4 *)(s_b(b, b_row) + 2 * b_half * 32);
                dst[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                dst[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
                dst[2] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                dst[3] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
                s_bd[b][b_row][2 * b_half] = __fmul_rn(d, (float)(scp & 0xFFu));
                s_bd[b][b_row][2 * b_half + 1] = __fmul_rn(d, (float)((scp >> 8) & 0xFFu));
                s_bm[b][b_row][2 * b_half] = -__fmul_rn(dmin, (float)(mnp & 0xFFu));
                s_bm[b][b_row][2 * b_half + 1] = -__fmul_rn(dmin, (float)((mnp >> 8) & 0xFFu));
                continue;
            }
#pragma unroll
            for (int hh = 0; hh < NBLK; hh++) {
                // the block this pass stages: block `blk` (0 .. 2 KS - 1) of the stage
                const int half = KS == 1 ? b_half : hh, blk = KS == 1 ? b_half : 2 * b_half + hh;
                uint32_t q[8];
                float sc, sc1, nm;
                expand_q<WT>(rb[b][NRAW == 2 ? hh : 0], k0 + (KS == 1 ? 0 : kBK * b_half), half, q, sc, sc1, nm);
                uint4 *dst = (uint4 *)(s_b(b, b_row) + blk * 32);
                dst[0] = make_uint4(q[0], q[1], q[2], q[3]);
                dst[1] = make_uint4(q[4], q[5], q[6], q[7]);
                if (SUB16) {
                    s_bd[b][b_row][2 * blk] = sc;
                    s_bd[b][b_row][2 * blk + 1] = sc1;
                } else {
                    s_bd[b][b_row][blk] = sc;
                }
                if (OFFSET) s_bm[b][b_row][blk] = nm;
            }
        }
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) *(uint4 *)(s_a(a_plane, a_row[p]) + a_chunk * 16) = ra[p];
        if (tid < KS * BM) s_as[tid / BM][tid % BM] = ras;
        if (OFFSET && tid < 2 * KS * BM) s_am[tid / (2 * KS)][tid & (2 * KS - 1)] = ram;
    };
    auto multiply = [&]() {
        // multiply: wave owns columns 32*wave .. +31
#pragma unroll
        for (int sub = 0; sub < KS; sub++) {
        if constexpr (!SUB16) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const int4v bq0 = *(const int4v *)(s_b(b, col) + 64 * sub + 16 * g);
                const int4v bq1 = *(const int4v *)(s_b(b, col) + 64 * sub + 32 + 16 * g);
                const float d0 = s_bd[b][col][2 * sub], d1 = s_bd[b][col][2 * sub + 1];
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const int arow = 32 * m + (lane & 31);
                    const int4v ah0 = *(const int4v *)(s_a(0, arow) + 64 * sub + 16 * g), al0 = *(const int4v *)(s_a(1, arow) + 64 * sub + 16 * g);
                    const int4v ah1 = *(const int4v *)(s_a(0, arow) + 64 * sub + 32 + 16 * g), al1 = *(const int4v *)(s_a(1, arow) + 64 * sub + 32 + 16 * g);
                    const int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const int16v ch0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ah0, bq0, zero, 0, 0, 0);
                    const int16v cl0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(al0, bq0, zero, 0, 0, 0);
                    const int16v ch1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ah1, bq1, zero, 0, 0, 0);
                    const int16v cl1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(al1, bq1, zero, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        // accumulator rows 8j..8j+7 of this 32-row block: past the tile's rows there is
                        // nothing to scale (ragged experts leave most of a tile empty at small batches)
                        if (GATE_UP && 32 * m + 8 * j >= rows) continue;  // (the down kernel measures faster without the test)
                        const float4 s4 = *(const float4 *)&s_as[sub][32 * m + 8 * j + 4 * g];
                        const float sr[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int r = 4 * j + i;
                            const float f0 = (float)((ch0[r] << 8) + cl0[r]);
                            const float f1 = (float)((ch1[r] << 8) + cl1[r]);
                            const float t = fmaf(d1, f1, __fmul_rn(d0, f0));
                            acc[b][m][r] = fmaf(t, sr[i], acc[b][m][r]);
                        }
                    }
                    if (OFFSET)
                        acc[b][m] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_am[arow][2 * sub + g], s_bm[b][col][2 * sub + g], acc[b][m], 0, 0, 0);
                }
            }
        }
        }
    };
    constexpr int STEP = KS * kBK;
    fetch(0);
    for (int k0 = 0; k0 < in_dim; k0 += STEP) {
        MUMMU_TIMER_MARK(0);
        stage(k0);
        MUMMU_TIMER_MARK(1);
        __syncthreads();
        MUMMU_TIMER_MARK(2);
        if (k0 + STEP < in_dim) fetch(k0 + STEP);
        MUMMU_TIMER_MARK(3);
        if constexpr (SUB16) {
            // (written out here, not in a lambda like the products of the other types: in a lambda this form
            // compiles to half as many more registers, spills for gate/up, and measures 10 % slower)
#pragma unroll
            for (int sub = 0; sub < KS; sub++) {
            // one weight scale per 16 elements: the K step is four 16-deep integer products
#pragma unroll
            for (int b = 0; b < NB; b++) {
                long bq[4];
                float dj[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    bq[j] = *(const long *)(s_b(b, col) + 64 * sub + 16 * j + 8 * g);
                    dj[j] = s_bd[b][col][4 * sub + j];
                }
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const int arow = 32 * m + (lane & 31);
                    float t[16] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const long ah = *(const long *)(s_a(0, arow) + 64 * sub + 16 * j + 8 * g), al = *(const long *)(s_a(1, arow) + 64 * sub + 16 * j + 8 * g);
                        const int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        const int16v ch = __builtin_amdgcn_mfma_i32_32x32x16_i8(ah, bq[j], zero, 0, 0, 0);
                        const int16v cl = __builtin_amdgcn_mfma_i32_32x32x16_i8(al, bq[j], zero, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            if (GATE_UP && 32 * m + 8 * (r >> 2) >= rows) continue;  // rows past the tile's: nothing to scale
                            const float f = (float)((ch[r] << 8) + cl[r]);
                            t[r] = j == 0 ? __fmul_rn(dj[0], f) : fmaf(dj[j], f, t[r]);
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const float4 s4 = *(const float4 *)&s_as[sub][32 * m + 8 * j + 4 * g];
                        const float sr[4] = {s4.x, s4.y, s4.z, s4.w};
                        if (!GATE_UP || 32 * m + 8 * j < rows) {
#pragma unroll
                            for (int i = 0; i < 4; i++) acc[b][m][4 * j + i] = fmaf(t[4 * j + i], sr[i], acc[b][m][4 * j + i]);
                        }
                    }
                }
            }
            }
        } else {
            multiply();
        }
        MUMMU_TIMER_MARK(4);
        __syncthreads();
        MUMMU_TIMER_MARK(5);
    }
    MUMMU_TIMER_STORE;

    if (GATE_UP) {
        // stage silu(g)*u of the whole tile as f32 (over the A and B tiles, no longer needed),
        // then quantize it in 64-element blocks
        float *s_c = (float *)s_raw;
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                s_c[(32 * m + acc_row(r, lane)) * kLdsC + col] = __fmul_rn(det_silu(acc[0][m][r]), acc[NB - 1][m][r]);
        __syncthreads();
        const int grp = tid >> 4, l16 = tid & 15;
#pragma unroll
        for (int pass = 0; pass < BM / 8; pass++) {
            const int task = pass * 16 + grp, row = task >> 1, cb = task & 1;
            const float4 v = *(const float4 *)&s_c[row * kLdsC + cb * 64 + 4 * l16];
            const bool active = row < rows && n0 + cb * 64 < out_dim;
            quantize_store64(active ? v : make_float4(0.f, 0.f, 0.f, 0.f), active, act_out, (size_t)(p0 + row), out_dim,
                             n0 + cb * 64 + 4 * l16);
        }
    } else {
        const int n = n0 + col;
        if (n < out_dim) {
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = 32 * m + acc_row(r, lane);
                    if (row < rows) y_out[(size_t)(p0 + row) * (size_t)out_dim + (size_t)n] = acc[0][m][r];
                }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Q4_K banks on the f16 units
// ---------------------------------------------------------------------------------------
// A Q4_K weight is d * (sc * q) - dmin * m with q < 16 and sc, m < 64 per 32 elements and d, dmin per 256.
// sc * q < 1024 is an exact half, so the matrix cores can sum x * (sc * q) over a whole run of
// sub-blocks with no vector work in between; the f32 accumulator takes d * that sum once per 128
// elements.  Activations come as pairs of halfs (HAct): the two products of a K step go into the
// same accumulator.  The offset term is one more instruction per 128 elements: the sums of the four
// 32-element blocks (hi and lo halfs, K = 8) against the four m.  Per output element and 128 elements
// of K that leaves three vector operations where the int8 form spends fourteen.

// Only the activation tile goes through LDS.  Wave w owns output columns 32w..32w+31 for every row of the
// tile, so the weights of those columns are its own: lane (column c, K group g) reads 16 of the 32 quant
// bytes of a 64-element step of row c straight into registers (low nibbles: elements 16g..16g+15, high
// nibbles: 32+16g..), turns them into its four B operands and never stores them anywhere.  The K index of
// an instruction therefore maps to element (kk/2)*32 + 16g + (kk%2)*8 + i of the step, and the A operands
// are read from the tile at that offset.  The activation tile is double-buffered (one barrier per step),
// loads run two steps (weights) and one step (activations) ahead of their use.
template <bool GATE_UP, int MT>
struct HTileLds {
    static constexpr int BM = 32 * MT;
    static constexpr int kRow = 2 * kLds;                     // LDS row (bytes): 64 halfs + 8 of padding
    static constexpr int kBuf = 2 * BM * kRow;                // hi and lo planes of one K step
    static constexpr int kC = GATE_UP ? BM * kLdsC * 4 : 0;   // f32 staging of the epilogue (aliases the tiles)
    static constexpr int kBytes = 2 * kBuf > kC ? 2 * kBuf : kC;
};

// GATE_UP: A = the token rows of a_in gathered through `sorted`; the epilogue writes silu(g)*u in sorted
//          order, as HAct (OUT_H: the down banks are Q4_K too) or in the int8 kernels' QAct64.
// else   : A = a_in rows in sorted order; y[pos, n] = f32 sum.
// WM: the workgroup has 4 WM waves; wave w owns columns 32 (w % 4) .. +31 of row blocks (w / 4) * MT / WM .. of the
// tile.  With two waves to a column block each expands the weights of its columns itself (twice the vector work
// in the workgroup) and keeps half the accumulators, which is what lets two workgroups share a CU without spills.
template <bool GATE_UP, int MT, int WM, bool OUT_H>
__global__ __launch_bounds__(256 * WM, GATE_UP ? 2 : 3) void grouped_gemm_q4k_f16_kernel(
    const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, HAct a_in, const int32_t *__restrict__ sorted, int k_slots,
    const int32_t *__restrict__ tiles, const int32_t *__restrict__ n_tiles, int in_dim, int out_dim, HAct act_h, QAct64 act_q,
    float *__restrict__ y_out) {
    using L = HTileLds<GATE_UP, MT>;
    constexpr int NB = GATE_UP ? 2 : 1, BM = L::BM, kRow = L::kRow;
    constexpr int MW = MT / WM, NT = 256 * WM;   // row blocks per wave, threads
    static_assert(MT % WM == 0, "row blocks split evenly over the wave rows");
    __shared__ __attribute__((aligned(16))) uint8_t s_raw[L::kBytes];
    __shared__ __attribute__((aligned(16))) float s_as[2][BM];         // activation scale of a 128-element run, per tile row
    __shared__ __attribute__((aligned(16))) _Float16 s_sum[2][BM][GATE_UP ? 16 : 8];   // block sums of one fold: hi halfs, then lo halfs
    auto s_a = [&](int buf, int plane, int row) -> _Float16 * {
        return (_Float16 *)(s_raw + (size_t)buf * L::kBuf + ((size_t)plane * BM + row) * kRow);
    };

    int tile, slab;
    if (!xcd_tile(n_tiles, (out_dim + kBN - 1) / kBN, tile, slab)) return;
    const int e = tiles[3 * tile], p0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = slab * kBN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t row_bytes = gemm_row_bytes(T_Q4_K, in_dim);
    const int col = 32 * (wave & 3) + (lane & 31), g = lane >> 5;
    const int row0 = 32 * MW * (wave >> 2);   // first tile row of this wave

    // Addresses are a uniform base plus a 32-bit byte offset per lane (an expert's bank and the activation planes
    // are far below 4 GB).  Rows past the tile's end read its last row and columns past the matrix its last column:
    // their products are never stored.
    const int b_out = n0 + col < out_dim ? n0 + col : out_dim - 1;
    const uint8_t *b_base[NB];
    b_base[0] = w0 + (size_t)e * (size_t)out_dim * row_bytes;
    if (GATE_UP) b_base[NB - 1] = w1 + (size_t)e * (size_t)out_dim * row_bytes;
    const uint32_t b_off = (uint32_t)b_out * (uint32_t)row_bytes + 16u * (uint32_t)g;

    auto source_row = [&](int r) -> int {
        r = r < rows ? r : rows - 1;
        return GATE_UP ? sorted[p0 + r] / k_slots : p0 + r;
    };
    // activation tile: thread -> (plane, row, 8 halfs), passes of 16 WM rows
    constexpr int A_PASSES = 2 * MT / WM, A_ROWS = 16 * WM;
    const int a_plane = tid / (NT / 2), a_chunk = tid & 7;
    const uint8_t *a_base = (const uint8_t *)(a_plane ? a_in.lo : a_in.hi);
    uint32_t a_off[A_PASSES], a_lds[A_PASSES];
#pragma unroll
    for (int p = 0; p < A_PASSES; p++) {
        const int r = A_ROWS * p + ((tid >> 3) & (A_ROWS - 1));
        a_off[p] = ((uint32_t)source_row(r) * (uint32_t)in_dim + (uint32_t)a_chunk * 8u) * 2u;
        a_lds[p] = (uint32_t)(((size_t)a_plane * BM + r) * kRow + a_chunk * 16);
    }
    // Activation scales.  ROW (the gate/up side: x comes from quantize_rows_h, one scale for the whole row): the
    // scale is applied once, in the epilogue, and a super-block is folded into acc in one go.  Otherwise (the down
    // side: the gate/up epilogue knows only its own 128 columns) every 128-element run has its own scale and is
    // folded on its own.
    // Block sums: thread -> (row tid / 4 of the tile, quarter tid % 4 of the run's blocks).  Threads past 4 BM
    // repeat rows and all four threads of a row store its scale: the same values twice, and no branch in the
    // loop body - with basic blocks in it the compiler sinks one step's arithmetic into the next and keeps both
    // steps' accumulators alive.
    constexpr bool ROW = GATE_UP;
    constexpr int NSUM = ROW ? 8 : 4;          // block sums per fold
    const int m_row = (tid >> 2) & (BM - 1), m_blk = tid & 3;
    const uint32_t src_m = (uint32_t)source_row(m_row);
    const uint32_t sum_off = (src_m * (uint32_t)(in_dim / 32) + (uint32_t)m_blk * (ROW ? 2u : 1u)) * 4u;
    const uint32_t scale_off = src_m * (uint32_t)(in_dim / 128) * 4u;
    if (ROW) s_as[0][m_row] = *(const float *)((const uint8_t *)a_in.scale + scale_off);

    float16v acc[NB][MW], c1[NB][MW];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int m = 0; m < MW; m++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[b][m][r] = c1[b][m][r] = 0.0f;

    // weights: the raw bytes of the step being multiplied and of the next one; of the current super-block d | dmin
    // and its eight scales and eight offsets as bytes (sub-blocks 0-3, 4-7); the header of the next super-block
    // during this one's last step
    u32x4 raw[2][NB], rh_next[NB];
    uint32_t dd[NB], sc4[NB][2], mn4[NB][2];
    // (the header of the NEXT super-block comes with the weights of this one's last step and is unpacked at the end
    // of that step, a whole step after its load: a value loaded in the loop's last step and first read in the next
    // iteration is copied between registers at the loop's end, behind a wait for every load in flight)
    auto load_b = [&](int k0, int st, u32x4 (&dst)[NB]) {
        const uint32_t o = b_off + (uint32_t)(k0 >> 8) * 144u;
        const uint32_t oh = b_off - 16u * (uint32_t)g + (k0 + 256 < in_dim ? (uint32_t)(k0 >> 8) * 144u + 144u : 0u);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            dst[b] = *(const u32x4 *)(b_base[b] + (o + 16u + (uint32_t)st * 32u));
            if (st == 3) rh_next[b] = *(const u32x4 *)(b_base[b] + oh);
        }
    };
    // ggml get_scale_min_k4 for all eight sub-blocks at once
    auto unpack_header = [&]() {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t y = rh_next[b][1], z = rh_next[b][2], w = rh_next[b][3];
            dd[b] = rh_next[b][0];
            sc4[b][0] = y & 0x3F3F3F3Fu;
            mn4[b][0] = z & 0x3F3F3F3Fu;
            sc4[b][1] = (w & 0x0F0F0F0Fu) | ((y >> 2) & 0x30303030u);
            mn4[b][1] = ((w >> 4) & 0x0F0F0F0Fu) | ((z >> 2) & 0x30303030u);
        }
    };
    // activations of one step in registers, then into a tile
    u32x4 ra[A_PASSES];
    float rsum[ROW ? 2 : 1] = {}, rscale = 0.0f;
    auto load_a = [&](int k0, int st) {
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) ra[p] = *(const u32x4 *)(a_base + (a_off[p] + (uint32_t)k0 * 2u));
        if (ROW) {
            if (st == 0) {
                const float2 v = *(const float2 *)((const uint8_t *)a_in.ssum + (sum_off + (uint32_t)(k0 >> 5) * 4u));
                rsum[0] = v.x;
                rsum[ROW ? 1 : 0] = v.y;
            }
        } else if ((st & 1) == 0) {
            rsum[0] = *(const float *)((const uint8_t *)a_in.ssum + (sum_off + (uint32_t)(k0 >> 5) * 4u));
            rscale = *(const float *)((const uint8_t *)a_in.scale + (scale_off + (uint32_t)(k0 >> 7) * 4u));
        }
    };
    // sum_buf: which of the two sets of block sums (they alternate per fold)
    auto store_a = [&](int buf, int st, int sum_buf) {
#pragma unroll
        for (int p = 0; p < A_PASSES; p++) *(u32x4 *)(s_raw + (size_t)buf * L::kBuf + a_lds[p]) = ra[p];
        if (ROW) {
            if (st == 0) {
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const float v = rsum[ROW ? i : 0];
                    const _Float16 h = (_Float16)v;
                    s_sum[sum_buf][m_row][2 * m_blk + i] = h;
                    s_sum[sum_buf][m_row][8 + 2 * m_blk + i] = (_Float16)__fsub_rn(v, (float)h);
                }
            }
        } else if ((st & 1) == 0) {
            const _Float16 h = (_Float16)rsum[0];
            s_sum[sum_buf][m_row][m_blk] = h;
            s_sum[sum_buf][m_row][4 + m_blk] = (_Float16)__fsub_rn(rsum[0], (float)h);
            s_as[sum_buf][m_row] = rscale;
        }
    };

    const float16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    // one 64-element step: st = which step of the super-block, buf = which tile holds its activations
    auto multiply = [&](int st, int buf, const u32x4 (&rw)[NB]) {
        half2v ml2[NB], al2[NB], mh2[NB], ah2[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) {
            // sub-blocks 2 st (the low nibbles) and 2 st + 1 (the high nibbles)
            const uint32_t sw = sc4[b][st >> 1] >> (16 * (st & 1));
            const float sc_lo = (float)(sw & 0xFFu), sc_hi = (float)((sw >> 8) & 0xFFu);
            // low nibbles: (1024 + q) * sc - 1024 sc; high nibbles, left in place: (1024 + 16 q) * (sc / 16) - 64 sc
            const _Float16 ml = (_Float16)sc_lo, al = (_Float16)__fmul_rn(-1024.0f, sc_lo);
            const _Float16 mh = (_Float16)__fmul_rn(0.0625f, sc_hi), ah = (_Float16)__fmul_rn(-64.0f, sc_hi);
            ml2[b] = half2v{ml, ml};
            al2[b] = half2v{al, al};
            mh2[b] = half2v{mh, mh};
            ah2[b] = half2v{ah, ah};
        }
        const uint8_t *tile = s_raw + (size_t)buf * L::kBuf + (size_t)(row0 + (lane & 31)) * kRow + 32 * g;
        // the A operands of instruction group kk + 1 are read from the tile before group kk is issued
        half8 a_hi[2][MW], a_lo[2][MW];
        auto read_a = [&](int kk) {
            const int a_byte = (kk >> 1) * 64 + (kk & 1) * 16;  // element (kk/2)*32 + 16g + (kk%2)*8 of the step
#pragma unroll
            for (int m = 0; m < MW; m++) {
                a_hi[kk & 1][m] = *(const half8 *)(tile + (size_t)(32 * m) * kRow + a_byte);
                a_lo[kk & 1][m] = *(const half8 *)(tile + (size_t)(BM + 32 * m) * kRow + a_byte);
            }
        };
        const bool first = ROW ? st == 0 : (st & 1) == 0;   // the step that starts a new sum in c1
        read_a(0);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (kk < 3) read_a(kk + 1);
            half8 bfrag[NB];
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const uint32_t w_a = (kk & 1) ? rw[b][2] : rw[b][0], w_b = (kk & 1) ? rw[b][3] : rw[b][1];
                const uint32_t mask = kk < 2 ? 0x0F0F0F0Fu : 0xF0F0F0F0u;
                const half2v mul = kk < 2 ? ml2[b] : mh2[b], add = kk < 2 ? al2[b] : ah2[b];
                half2v f[4];
                f[0] = __builtin_elementwise_fma(biased_pair(w_a & mask, false), mul, add);
                f[1] = __builtin_elementwise_fma(biased_pair(w_a & mask, true), mul, add);
                f[2] = __builtin_elementwise_fma(biased_pair(w_b & mask, false), mul, add);
                f[3] = __builtin_elementwise_fma(biased_pair(w_b & mask, true), mul, add);
                __builtin_memcpy(&bfrag[b], f, 16);
            }
            // (the hi products of every block first, then the lo products: instructions that accumulate into the same
            // registers are NB * MW apart)
#pragma unroll
            for (int m = 0; m < MW; m++)
#pragma unroll
                for (int b = 0; b < NB; b++)
                    c1[b][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_hi[kk & 1][m], bfrag[b], (first && kk == 0) ? zero : c1[b][m], 0, 0, 0);
#pragma unroll
            for (int m = 0; m < MW; m++)
#pragma unroll
                for (int b = 0; b < NB; b++)
                    c1[b][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_lo[kk & 1][m], bfrag[b], c1[b][m], 0, 0, 0);
        }
    };
    // what has been summed into c1 -> acc.  part: which 128-element run of the super-block (the whole of it with
    // one scale per row); sum_buf: which set of block sums
    auto fold = [&](int part, int sum_buf) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float d = half_bits_to_float((uint16_t)(dd[b] & 0xFFFFu));
            const float ndmin = -half_bits_to_float((uint16_t)(dd[b] >> 16));
            // the block offsets m as halfs (exact), in the order of the block sums
            _Float16 mh[NSUM];
#pragma unroll
            for (int j = 0; j < NSUM; j++) {
                const uint32_t word = ROW ? mn4[b][j >> 2] : mn4[b][part];
                mh[j] = (_Float16)(float)((word >> (8 * (j & 3))) & 0xFFu);
            }
#pragma unroll
            for (int m = 0; m < MW; m++) {
                float16v c2;
                if constexpr (ROW) {
                    // K = 16: the eight sums' hi halfs from lanes 0-31, their lo halfs from lanes 32-63
                    const half8 am = *(const half8 *)&s_sum[sum_buf][row0 + 32 * m + (lane & 31)][8 * g];
                    half8 bm;
#pragma unroll
                    for (int j = 0; j < 8; j++) bm[j] = mh[j];
                    c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[b][m][r] = fmaf(ndmin, c2[r], fmaf(d, c1[b][m][r], acc[b][m][r]));
                } else {
                    const half4v am = *(const half4v *)&s_sum[sum_buf][row0 + 32 * m + (lane & 31)][4 * g];
                    const half4v bm = {mh[0], mh[1], mh[2], mh[3]};
                    c2 = __builtin_amdgcn_mfma_f32_32x32x8f16(am, bm, zero, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const float4 s4 = *(const float4 *)&s_as[sum_buf][row0 + 32 * m + 8 * j + 4 * g];
                        const float sr[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int r = 4 * j + i;
                            const float u = fmaf(ndmin, c2[r], __fmul_rn(d, c1[b][m][r]));
                            acc[b][m][r] = fmaf(u, sr[i], acc[b][m][r]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // (one 32 x 32 block at a time: scheduled together they do not fit the registers)
            }
        }
    };

    // prologue: the first header, step 0 into tile 0
#pragma unroll
    for (int b = 0; b < NB; b++) rh_next[b] = *(const u32x4 *)(b_base[b] + (b_off - 16u * (uint32_t)g));
    unpack_header();
    load_b(0, 0, raw[0]);
    load_a(0, 0);
    store_a(0, 0, 0);
    __syncthreads();
    MUMMU_TIMER_DECL;
    // (one step as a generic lambda over a compile-time step index: the register sets are picked by constants)
    auto step = [&](int sb0, auto st_c) {
        constexpr int st = decltype(st_c)::value;
        // (after the last step the "next" one is step 0 again: loaded and stored like any other, never multiplied;
        // no branch in the loop body)
        const int k_next = (st == 3 && sb0 + 256 >= in_dim) ? 0 : sb0 + kBK * (st + 1);
        // block sums alternate between two sets: per super-block with one scale per row, else per 128-element run
        const int sb_par = (sb0 >> 8) & 1;
        const int sum_buf = ROW ? sb_par : (st >> 1) & 1;
        const int sum_buf_next = ROW ? (st == 3 ? sb_par ^ 1 : sb_par) : (((st + 1) & 3) >> 1) & 1;
        MUMMU_TIMER_MARK(0);
        // the next step: activations into registers, weights into the other set of registers.  (Loads come back in
        // the order issued: the activations are wanted at the end of this step, the weights a step later, so the
        // wait before store_a must not have the weight loads in front of it.)
        load_a(k_next, (st + 1) & 3);
        load_b(k_next, (st + 1) & 3, raw[(st + 1) & 1]);
        MUMMU_CODE_FENCE();  // (the loads stay here, a whole step ahead of their first use)
        MUMMU_TIMER_MARK(1);
        multiply(st, st & 1, raw[st & 1]);
        MUMMU_TIMER_MARK(2);
        if (ROW ? st == 3 : (st & 1) == 1) fold(st >> 1, sum_buf);
        if (st == 3) unpack_header();
        MUMMU_TIMER_MARK(3);
        MUMMU_CODE_FENCE();
        // ... and into the tile that the step before this one was read from
        store_a((st + 1) & 1, (st + 1) & 3, sum_buf_next);
        MUMMU_TIMER_MARK(4);
        __syncthreads();
        MUMMU_TIMER_MARK(5);
    };
    for (int sb0 = 0; sb0 < in_dim; sb0 += 256) {
        step(sb0, std::integral_constant<int, 0>{});
        step(sb0, std::integral_constant<int, 1>{});
        step(sb0, std::integral_constant<int, 2>{});
        step(sb0, std::integral_constant<int, 3>{});
    }
    MUMMU_TIMER_STORE;

    if (GATE_UP) {
        // stage silu(g)*u of the whole tile as f32 (over the activation tiles, no longer needed), then store it in the
        // form the down product reads
        float *s_c = (float *)s_raw;
#pragma unroll
        for (int m = 0; m < MW; m++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                // (one scale per row on this side: both products take it here)
                const float sr = s_as[0][row0 + 32 * m + acc_row(r, lane)];
                s_c[(row0 + 32 * m + acc_row(r, lane)) * kLdsC + col] =
                    __fmul_rn(det_silu(__fmul_rn(sr, acc[0][m][r])), __fmul_rn(sr, acc[NB - 1][m][r]));
            }
        __syncthreads();
        if (OUT_H) {
            const int grp = tid >> 5, l32 = tid & 31;
#pragma unroll
            for (int pass = 0; pass < BM / (NT / 32); pass++) {
                const int row = pass * (NT / 32) + grp;
                const float4 v = *(const float4 *)&s_c[row * kLdsC + 4 * l32];
                const bool active = row < rows && n0 < out_dim;
                hact_store128(active ? v : make_float4(0.f, 0.f, 0.f, 0.f), active, act_h, (size_t)(p0 + row), out_dim, n0 + 4 * l32);
            }
        } else {
            const int grp = tid >> 4, l16 = tid & 15;
#pragma unroll
            for (int pass = 0; pass < 2 * BM / (NT / 16); pass++) {
                const int task = pass * (NT / 16) + grp, row = task >> 1, cb = task & 1;
                const float4 v = *(const float4 *)&s_c[row * kLdsC + cb * 64 + 4 * l16];
                const bool active = row < rows && n0 + cb * 64 < out_dim;
                quantize_store64(active ? v : make_float4(0.f, 0.f, 0.f, 0.f), active, act_q, (size_t)(p0 + row), out_dim,
                                 n0 + cb * 64 + 4 * l16);
            }
        }
    } else {
        const int n = n0 + col;
        if (n < out_dim) {
#pragma unroll
            for (int m = 0; m < MW; m++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = row0 + 32 * m + acc_row(r, lane);
                    if (row < rows) y_out[(size_t)(p0 + row) * (size_t)out_dim + (size_t)n] = acc[0][m][r];
                }
        }
    }
}

// The same product for experts with few rows (small batches): 16-row tiles on v_mfma_f32_16x16x32_f16.  Eight
// waves, wave w owns output columns 16w..16w+15; a stage is half a super-block (128 elements).  Lane (column c,
// K group kg) reads 16 of the 64 quant bytes of the stage - the four lanes of a column read 64 consecutive bytes
// of its row - and supplies, in instruction q of the stage, the eight elements
//     64 (kg / 2) + 16 (kg % 2) + 32 (q / 2) + 8 (q % 2) + 0..7
// (low nibbles of its bytes for q < 2, high nibbles after), and the activation operands are read from the tile at
// that offset.  A quarter of the accumulators and half the matrix work of the 32-row form, and twice the waves
// on a SIMD.
template <bool GATE_UP, bool OUT_H>
__global__ __launch_bounds__(512, 4) void grouped_gemm_q4k_f16_m16_kernel(
    const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, HAct a_in, const int32_t *__restrict__ sorted, int k_slots,
    const int32_t *__restrict__ tiles, const int32_t *__restrict__ n_tiles, int in_dim, int out_dim, HAct act_h, QAct64 act_q,
    float *__restrict__ y_out) {
    constexpr int NB = GATE_UP ? 2 : 1, BM = 16;
    constexpr int kRow = 2 * 128 + 16;                 // LDS row (bytes): 128 halfs + 16 bytes keep 16-byte reads conflict-free
    constexpr int kPlane = BM * kRow, kBuf = 2 * kPlane;   // hi plane, lo plane of one stage
    constexpr int kC = GATE_UP ? BM * kLdsC * 4 : 0;   // f32 staging of the epilogue (aliases the tiles)
    constexpr int kBytes = 2 * kBuf > kC ? 2 * kBuf : kC;
    constexpr bool ROW = GATE_UP;                      // one activation scale per row (else per 128 elements = per stage)
    __shared__ __attribute__((aligned(16))) uint8_t s_raw[kBytes];
    __shared__ __attribute__((aligned(16))) float s_as[2][BM];
    // block sums of one fold.  ROW: the super-block's eight hi halfs, then its eight lo halfs; else the stage's four
    // hi halfs, four lo halfs and eight zeros (the fold is one K = 16 instruction either way)
    // (rows of 20 halfs: with 16 the rows four apart share their banks)
    __shared__ __attribute__((aligned(16))) _Float16 s_sum[2][BM][20];

    int tile, slab;
    if (!xcd_tile(n_tiles, (out_dim + kBN - 1) / kBN, tile, slab)) return;
    const int e = tiles[3 * tile], p0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = slab * kBN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t row_bytes = gemm_row_bytes(T_Q4_K, in_dim);
    const int c = lane & 15, kg = lane >> 4;
    const int col = 16 * wave + c;

    const int b_out = n0 + col < out_dim ? n0 + col : out_dim - 1;
    const uint8_t *b_base[NB];
    b_base[0] = w0 + (size_t)e * (size_t)out_dim * row_bytes;
    if (GATE_UP) b_base[NB - 1] = w1 + (size_t)e * (size_t)out_dim * row_bytes;
    const uint32_t h_off = (uint32_t)b_out * (uint32_t)row_bytes;   // the row's first super-block header
    const uint32_t b_off = h_off + 16u + 16u * (uint32_t)kg;

    auto source_row = [&](int r) -> int {
        r = r < rows ? r : rows - 1;
        return GATE_UP ? sorted[p0 + r] / k_slots : p0 + r;
    };
    // activation tile: thread -> (plane, row, 8 halfs of the stage's 128)
    const int a_plane = tid >> 8, a_row = (tid >> 4) & 15, a_chunk = tid & 15;
    const uint8_t *a_base = (const uint8_t *)(a_plane ? a_in.lo : a_in.hi);
    const uint32_t a_off = ((uint32_t)source_row(a_row) * (uint32_t)in_dim + (uint32_t)a_chunk * 8u) * 2u;
    const uint32_t a_lds = (uint32_t)(a_plane * kPlane + a_row * kRow + a_chunk * 16);
    // block sums: thread -> (row, one of the stage's four blocks); every thread stores (threads past 64 repeat rows)
    const int m_row = (tid >> 2) & (BM - 1), m_blk = tid & 3;
    const uint32_t src_m = (uint32_t)source_row(m_row);
    const uint32_t sum_off = (src_m * (uint32_t)(in_dim / 32) + (uint32_t)m_blk) * 4u;
    const uint32_t scale_off = src_m * (uint32_t)(in_dim / 128) * 4u;
    if (ROW) s_as[0][m_row] = *(const float *)((const uint8_t *)a_in.scale + scale_off);
    if (!ROW) {
        s_sum[0][m_row][8 + m_blk] = s_sum[0][m_row][12 + m_blk] = (_Float16)0.0f;
        s_sum[1][m_row][8 + m_blk] = s_sum[1][m_row][12 + m_blk] = (_Float16)0.0f;
    }

    f32x4 acc[NB], c1[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) acc[b] = c1[b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4 raw[2][NB], rh_next[NB];
    uint32_t dd[NB], sc4[NB][2], mn4[NB][2];
    auto load_b = [&](int k0, u32x4 (&dst)[NB]) {
        const uint32_t o = b_off + (uint32_t)(k0 >> 8) * 144u + (uint32_t)((k0 >> 7) & 1) * 64u;
#pragma unroll
        for (int b = 0; b < NB; b++) dst[b] = *(const u32x4 *)(b_base[b] + o);
    };
    auto load_header = [&](int k0) {
#pragma unroll
        for (int b = 0; b < NB; b++) rh_next[b] = *(const u32x4 *)(b_base[b] + (h_off + (uint32_t)(k0 >> 8) * 144u));
    };
    auto unpack_header = [&]() {   // ggml get_scale_min_k4 for all eight sub-blocks at once
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t y = rh_next[b][1], z = rh_next[b][2], w = rh_next[b][3];
            dd[b] = rh_next[b][0];
            sc4[b][0] = y & 0x3F3F3F3Fu;
            mn4[b][0] = z & 0x3F3F3F3Fu;
            sc4[b][1] = (w & 0x0F0F0F0Fu) | ((y >> 2) & 0x30303030u);
            mn4[b][1] = ((w >> 4) & 0x0F0F0F0Fu) | ((z >> 2) & 0x30303030u);
        }
    };
    u32x4 ra;
    float rsum = 0.0f, rscale = 0.0f;
    auto load_a = [&](int k0) {
        ra = *(const u32x4 *)(a_base + (a_off + (uint32_t)k0 * 2u));
        rsum = *(const float *)((const uint8_t *)a_in.ssum + (sum_off + (uint32_t)(k0 >> 5) * 4u));
        if (!ROW) rscale = *(const float *)((const uint8_t *)a_in.scale + (scale_off + (uint32_t)(k0 >> 7) * 4u));
    };
    // buf: the tile of the stage; sum_buf / slot: where its block sums go
    auto store_a = [&](int buf, int sum_buf, int slot) {
        *(u32x4 *)(s_raw + (size_t)buf * kBuf + a_lds) = ra;
        if (wave == 0) {   // (every wave holds the same sums: one stores them)
            const _Float16 h = (_Float16)rsum;
            s_sum[sum_buf][m_row][slot + m_blk] = h;
            s_sum[sum_buf][m_row][slot + (ROW ? 8 : 4) + m_blk] = (_Float16)__fsub_rn(rsum, (float)h);
            if (!ROW) s_as[sum_buf][m_row] = rscale;
        }
    };

    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    auto multiply = [&](int hs, int buf, const u32x4 (&rw)[NB], bool first) {
        half2v ml2[NB], al2[NB], mh2[NB], ah2[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) {
            // this lane's bytes belong to sub-blocks 4 hs + 2 (kg / 2) (low nibbles) and the one after (high nibbles)
            // (hs is a constant at every call: picked with a conditional, an index would send the array to LDS)
            const uint32_t sw = (hs ? sc4[b][1] : sc4[b][0]) >> (16 * (kg >> 1));
            const float sc_lo = (float)(sw & 0xFFu), sc_hi = (float)((sw >> 8) & 0xFFu);
            const _Float16 ml = (_Float16)sc_lo, al = (_Float16)__fmul_rn(-1024.0f, sc_lo);
            const _Float16 mh = (_Float16)__fmul_rn(0.0625f, sc_hi), ah = (_Float16)__fmul_rn(-64.0f, sc_hi);
            ml2[b] = half2v{ml, ml};
            al2[b] = half2v{al, al};
            mh2[b] = half2v{mh, mh};
            ah2[b] = half2v{ah, ah};
        }
        const uint8_t *tile_p = s_raw + (size_t)buf * kBuf + (size_t)(lane & 15) * kRow + 128 * (kg >> 1) + 32 * (kg & 1);
        half8 a_hi[2], a_lo[2];
        auto read_a = [&](int q) {
            const int a_byte = 64 * (q >> 1) + 16 * (q & 1);
            a_hi[q & 1] = *(const half8 *)(tile_p + a_byte);
            a_lo[q & 1] = *(const half8 *)(tile_p + kPlane + a_byte);
        };
        read_a(0);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (q < 3) read_a(q + 1);
            half8 bfrag[NB];
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const uint32_t w_a = (q & 1) ? rw[b][2] : rw[b][0], w_b = (q & 1) ? rw[b][3] : rw[b][1];
                const uint32_t mask = q < 2 ? 0x0F0F0F0Fu : 0xF0F0F0F0u;
                const half2v mul = q < 2 ? ml2[b] : mh2[b], add = q < 2 ? al2[b] : ah2[b];
                half2v f[4];
                f[0] = __builtin_elementwise_fma(biased_pair(w_a & mask, false), mul, add);
                f[1] = __builtin_elementwise_fma(biased_pair(w_a & mask, true), mul, add);
                f[2] = __builtin_elementwise_fma(biased_pair(w_b & mask, false), mul, add);
                f[3] = __builtin_elementwise_fma(biased_pair(w_b & mask, true), mul, add);
                __builtin_memcpy(&bfrag[b], f, 16);
            }
#pragma unroll
            for (int b = 0; b < NB; b++)
                c1[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi[q & 1], bfrag[b], (first && q == 0) ? zero : c1[b], 0, 0, 0);
#pragma unroll
            for (int b = 0; b < NB; b++) c1[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo[q & 1], bfrag[b], c1[b], 0, 0, 0);
        }
    };
    // what has been summed into c1 -> acc (hs: the stage, for the per-stage fold of the down side)
    auto fold = [&](int hs, int sum_buf) {
        const half4v am = *(const half4v *)&s_sum[sum_buf][lane & 15][4 * kg];
        float sr[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        if (!ROW) {
            const float4 s4 = *(const float4 *)&s_as[sum_buf][4 * kg];
            sr[0] = s4.x, sr[1] = s4.y, sr[2] = s4.z, sr[3] = s4.w;
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float d = half_bits_to_float((uint16_t)(dd[b] & 0xFFFFu));
            const float ndmin = -half_bits_to_float((uint16_t)(dd[b] >> 16));
            // K index 4 kg + i of the fold: sub-block (4 kg + i) % 8 with ROW, else 4 hs + i (its K groups 2, 3 meet zeros)
            // (with one scale per row the word depends on the lane: blended with a mask - a conditional between the two
            // array elements becomes an indexed load and sends the array to LDS)
            const uint32_t lane_mask = 0u - (uint32_t)(kg & 1);
            const uint32_t word = ROW ? (mn4[b][0] ^ ((mn4[b][0] ^ mn4[b][1]) & lane_mask)) : (hs ? mn4[b][1] : mn4[b][0]);
            half4v bm;
#pragma unroll
            for (int i = 0; i < 4; i++) bm[i] = (_Float16)(float)((word >> (8 * i)) & 0xFFu);
            const f32x4 c2 = __builtin_amdgcn_mfma_f32_16x16x16f16(am, bm, zero, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (ROW) {
                    acc[b][i] = fmaf(ndmin, c2[i], fmaf(d, c1[b][i], acc[b][i]));
                } else {
                    const float u = fmaf(ndmin, c2[i], __fmul_rn(d, c1[b][i]));
                    acc[b][i] = fmaf(u, sr[i], acc[b][i]);
                }
            }
        }
    };

    // prologue: the first header, stage 0 into tile 0
    load_header(0);
    unpack_header();
    load_a(0);
    load_b(0, raw[0]);
    store_a(0, 0, 0);
    __syncthreads();
    auto stage = [&](int sb0, auto hs_c) {
        constexpr int hs = decltype(hs_c)::value;
        // (after the last stage the "next" one is stage 0 again: loaded and stored like any other, never multiplied)
        const int sb_next = sb0 + 256 < in_dim ? sb0 + 256 : 0;
        const int k_next = hs == 0 ? sb0 + 128 : sb_next;
        const int sb_par = (sb0 >> 8) & 1;
        load_a(k_next);
        load_b(k_next, raw[(hs + 1) & 1]);
        if (hs == 0) load_header(sb_next);   // (a stage before its unpacking: nothing loaded in the loop's last stage is first read in the next iteration)
        MUMMU_CODE_FENCE();
        multiply(hs, hs, raw[hs], ROW ? hs == 0 : true);
        if (ROW ? hs == 1 : true) fold(hs, ROW ? sb_par : hs);
        if (hs == 1) unpack_header();
        MUMMU_CODE_FENCE();
        if (ROW) store_a((hs + 1) & 1, hs == 0 ? sb_par : sb_par ^ 1, hs == 0 ? 4 : 0);
        else store_a((hs + 1) & 1, (hs + 1) & 1, 0);
        __syncthreads();
    };
    for (int sb0 = 0; sb0 < in_dim; sb0 += 256) {
        stage(sb0, std::integral_constant<int, 0>{});
        stage(sb0, std::integral_constant<int, 1>{});
    }

    if (GATE_UP) {
        float *s_c = (float *)s_raw;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = 4 * kg + i;
            const float sr = s_as[0][row];   // (one scale per row on this side: both products take it here)
            s_c[row * kLdsC + col] = __fmul_rn(det_silu(__fmul_rn(sr, acc[0][i])), __fmul_rn(sr, acc[NB - 1][i]));
        }
        __syncthreads();
        if (OUT_H) {
            const int row = tid >> 5, l32 = tid & 31;
            const float4 v = *(const float4 *)&s_c[row * kLdsC + 4 * l32];
            const bool active = row < rows && n0 < out_dim;
            hact_store128(active ? v : make_float4(0.f, 0.f, 0.f, 0.f), active, act_h, (size_t)(p0 + row), out_dim, n0 + 4 * l32);
        } else {
            const int grp = tid >> 4, l16 = tid & 15, row = grp >> 1, cb = grp & 1;
            const float4 v = *(const float4 *)&s_c[row * kLdsC + cb * 64 + 4 * l16];
            const bool active = row < rows && n0 + cb * 64 < out_dim;
            quantize_store64(active ? v : make_float4(0.f, 0.f, 0.f, 0.f), active, act_q, (size_t)(p0 + row), out_dim,
                             n0 + cb * 64 + 4 * l16);
        }
    } else {
        const int n = n0 + col;
        if (n < out_dim) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = 4 * kg + i;
                if (row < rows) y_out[(size_t)(p0 + row) * (size_t)out_dim + (size_t)n] = acc[0][i];
            }
        }
    }
}

// x [n, d] f32 -> HAct with one scale per row: a workgroup per row finds the row's largest magnitude, then
// stores the row 1024 elements at a time.
__global__ __launch_bounds__(256) void quantize_rows_h_kernel(const float *__restrict__ x, int d, HAct q) {
    __shared__ float s_max[4];
    hact_quantize_row<256>(x, d, q, (int)blockIdx.x, s_max);
}

// x [n, d] f32 -> f16, round to nearest.
__global__ __launch_bounds__(256) void convert_rows_f16_kernel(const float *__restrict__ x, size_t count, _Float16 *__restrict__ out) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count) return;
    const float4 v = *(const float4 *)(x + i);
    *(uint2 *)(out + i) = make_uint2(pack_half2(v.x, v.y), pack_half2(v.z, v.w));
}

hipError_t launch_convert_rows_f16(const float *x, int n, int d, _Float16 *out, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (d % 4 != 0) return hipErrorInvalidValue;
    const size_t count = (size_t)n * (size_t)d;
    launch_kernel(convert_rows_f16_kernel, dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, s, x, count, out);
    return hipGetLastError();
}

hipError_t launch_quantize_rows_h(const float *x, int n, int d, HAct q, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (d % 128 != 0) return hipErrorInvalidValue;
    launch_kernel(quantize_rows_h_kernel, dim3(n), dim3(256), 0, s, x, d, q);
    return hipGetLastError();
}

// x [n, d] f32 -> QAct64: one 16-lane row per 64-element block.
__global__ __launch_bounds__(256) void quantize_rows64_kernel(const float *__restrict__ x, int d, QAct64 q) {
    const int row = blockIdx.y;
    const int elem0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    const bool active = elem0 < d;
    const float4 v = active ? *(const float4 *)(x + (size_t)row * (size_t)d + elem0) : make_float4(0.f, 0.f, 0.f, 0.f);
    quantize_store64(v, active, q, (size_t)row, d, elem0);
}

hipError_t launch_quantize_rows64(const float *x, int n, int d, QAct64 q, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (d % 64 != 0) return hipErrorInvalidValue;
    launch_kernel(quantize_rows64_kernel, dim3((d + 1023) / 1024, n), dim3(256), 0, s, x, d, q);
    return hipGetLastError();
}

static bool gemm_q_type(int t) { return is_quant_type(t); }

bool grouped_gemm_quantized(const ExpertBanks &b) {
    return gemm_q_type(b.gate_type) && b.gate_type == b.up_type && gemm_q_type(b.down_type);
}

bool grouped_gemm_supported(const ExpertBanks &b) {
    const bool f16 = (b.gate_type == T_F16 || b.gate_type == T_BF16 || b.gate_type == T_F32) && b.up_type == b.gate_type &&
                     b.down_type == b.gate_type;
    return (f16 || grouped_gemm_quantized(b)) && b.hidden % kBK == 0 && b.inter % kBK == 0;
}

// Rows per tile.  An expert with one row more than a tile holds runs a second, almost empty tile
// that streams its whole weight slab again, so the tile is sized to hold the average expert load
// plus its spread (binomial: about +-sqrt(avg) per expert, 3.5 sigma here) when that fits; the f16
// kernel goes up to 128 rows, the int8 kernel (more registers per row) to 64.
// Tile rows for the f16-unit Q4_K kernels, which come in 16-, 32- and 64-row forms: the one with the smallest
// expected cost when an expert's rows are spread like a binomial around the average (normal approximation,
// variance = mean).  A 32-row workgroup costs 0.55 of a 64-row one (measured at 4096 tokens, where both forms run
// full tiles): the expansion of the weights, the loads and the barriers do not shrink with the rows.  At an
// average of 64 rows half the experts need a second, almost empty 64-row tile and 32-row tiles win; at 48 one
// 64-row tile holds nearly every expert and wins; from a few hundred rows on the 64-row form wins by its 9 %.
// A launch of 16-row tiles costs 0.83-0.89 of one with as many 32-row tiles (32 / 64 tokens over 64 experts: gate/up
// 46.1 / 50.2 against 56.0 / 55.8 us, down 25.1 / 26.7 against 30.0 / 30.8 us), but every expert that needs a second
// tile streams its weights again: with 10 % more tiles (96 tokens) the 16-row launches already take 65.9 + 33.9 us
// against 56.5 + 31.8 us.  So the 16-row form is taken only while next to no expert has more than 16 rows (its
// expected tiles within 1 % of the 32-row form's: 64 experts x 8 slabs of 16-row tiles are exactly the 512
// workgroups the chip holds at once, and the first second tiles start a second round - 72 / 80 tokens: 104 / 114 us
// per layer with 16-row tiles, 105 / 106-112 us with 32-row tiles).
int grouped_gemm_tile_rows_q4k_f16(int n_assign, int n_experts) {
    const double avg = (double)n_assign / (double)(n_experts > 0 ? n_experts : 1);
    const double sigma = __builtin_sqrt(avg > 1.0 ? avg : 1.0);
    auto expected_tiles = [&](double rows) {
        double t = 0.0;
        for (int j = 0; j < 1024; j++) {
            const double p = 0.5 * erfc(((double)j * rows + 0.5 - avg) / (sigma * 1.4142135623730951));
            t += p;
            if (p < 1e-6) break;
        }
        return t;
    };
    const double e16 = expected_tiles(16.0), e32 = expected_tiles(32.0), e64 = expected_tiles(64.0);
    if (0.99 * e16 < e32 && 0.99 * 0.55 * e16 < e64) return 16;
    return 0.55 * e32 < e64 ? 32 : 64;
}

int grouped_gemm_tile_rows(const ExpertBanks &b, int n_assign, int n_experts, bool q8_half) {
    const int max_rows = ((grouped_gemm_quantized(b) && !q8_half) || b.gate_type == T_F32) ? 64 : 128;
    const double avg = (double)n_assign / (double)n_experts;
    const int want = (int)(avg + 3.5 * __builtin_sqrt(avg) + 1.0);
    if (want > max_rows) return 64;  // several full tiles per expert whatever the size: 64 rows measured best
    int rows = 32;
    while (rows < want) rows += 32;
    return rows;
}

template <int WT, bool GATE_UP>
static hipError_t launch_gemm_q(const uint8_t *w0, const uint8_t *w1, QAct64 a_in, const int32_t *sorted, int k_slots,
                                const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, bool few_rows,
                                int in_dim, int out_dim, QAct64 act_out, float *y_out, hipStream_t s) {
    dim3 block(256), grid((unsigned)((max_tiles + 7) / 8 * 8) * (unsigned)((out_dim + kBN - 1) / kBN));
    // Two K steps per stage where the row length allows and it measured faster: always for the types
    // whose one load holds both blocks of a step (Q4_K, Q5_K: no extra registers) and for gate/up;
    // the down product of the other types only while an expert's rows fit one tile (with several
    // tiles per expert its second set of raw registers costs more than the barriers saved: Q8_0 at
    // 4096 tokens 410 -> 462 us), and for Q6_K only with 32-row tiles (32 tokens 84 -> 72 us, but 512
    // tokens 138 -> 142 us).
    constexpr bool shared_raw = WT == T_Q4_K || WT == T_Q5_K;
    const bool ks2 = in_dim % (2 * kBK) == 0 && (shared_raw || GATE_UP || few_rows) && !(gemm_sub16(WT) && !GATE_UP && tile_rows == 64);
#define MUMMU_Q(MT, KS)                                                                                             \
    launch_kernel(grouped_gemm_q_kernel<WT, GATE_UP, MT, KS>, grid, block, 0, s, w0, w1, a_in, sorted, k_slots, tiles,   \
                  n_tiles, in_dim, out_dim, act_out, y_out)
    // small tiles (few rows per expert: the launch is a stream of weights) also keep two stages of loads in flight
    if (tile_rows == 64 && ks2) MUMMU_Q(2, 2);
    else if (tile_rows == 64) MUMMU_Q(2, 1);
    else if (ks2) MUMMU_Q(1, 2);
    else MUMMU_Q(1, 1);
#undef MUMMU_Q
    return hipGetLastError();
}

// Largest |d| of a Q8_0 bank as half bits (infinities and NaNs compare above every finite value).
__global__ __launch_bounds__(256) void q8_scale_max_kernel(const uint8_t *__restrict__ bank, size_t n_blocks, uint32_t *__restrict__ max_bits) {
    uint32_t m = 0u;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_blocks; i += (size_t)gridDim.x * 256) {
        uint16_t db;
        __builtin_memcpy(&db, bank + i * 34, 2);
        const uint32_t a = db & 0x7FFFu;
        m = a > m ? a : m;
    }
    m = (uint32_t)wave_max_i32((int)m);
    if ((threadIdx.x & 63) == 0 && m != 0u) atomicMax(max_bits, m);
}

hipError_t launch_q8_scale_max(const uint8_t *bank, size_t n_blocks, uint32_t *max_bits, hipStream_t s) {
    if (n_blocks == 0) return hipSuccess;
    const size_t want = (n_blocks + 255) / 256;
    launch_kernel(q8_scale_max_kernel, dim3((unsigned)(want < 2048 ? want : 2048)), dim3(256), 0, s, bank, n_blocks, max_bits);
    return hipGetLastError();
}

// Q8_0 banks through the f16 kernel (every weight as two halfs): all three banks Q8_0 and, checked when the layer
// was loaded, every |d| * 128 inside the half range
bool grouped_gemm_q8_f16(const ExpertBanks &b) {
    return b.q8_half_ok && b.gate_type == T_Q8_0 && b.up_type == T_Q8_0 && b.down_type == T_Q8_0 && b.hidden % 64 == 0 &&
           b.inter % 64 == 0;
}

bool grouped_gemm_q4k_f16(const ExpertBanks &b) {
    // (one expert's matrix is addressed with 32-bit byte offsets)
    return b.gate_type == T_Q4_K && b.up_type == T_Q4_K && b.hidden % 256 == 0 && b.inter % 128 == 0 &&
           (size_t)b.hidden * (size_t)b.inter < (1ull << 32);
}

bool grouped_gemm_q4k_f16_down(const ExpertBanks &b) {
    return grouped_gemm_q4k_f16(b) && b.down_type == T_Q4_K && b.inter % 256 == 0 && b.hidden % 128 == 0;
}

template <bool GATE_UP>
static hipError_t launch_gemm_q4k_f16(const uint8_t *w0, const uint8_t *w1, HAct a_in, const int32_t *sorted, int k_slots,
                                      const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, int in_dim,
                                      int out_dim, HAct act_h, QAct64 act_q, bool out_h, float *y_out, hipStream_t s) {
    dim3 grid((unsigned)((max_tiles + 7) / 8 * 8) * (unsigned)((out_dim + kBN - 1) / kBN));
#define MUMMU_H(MT, WM, OUT_H)                                                                                           \
    launch_kernel(grouped_gemm_q4k_f16_kernel<GATE_UP, MT, WM, OUT_H>, grid, dim3(256 * WM), 0, s, w0, w1, a_in, sorted, k_slots, \
                  tiles, n_tiles, in_dim, out_dim, act_h, act_q, y_out)
    if (tile_rows == 64) {
        if (out_h) MUMMU_H(2, 1, true);
        else MUMMU_H(2, 1, false);
    } else if (tile_rows == 32) {
        if (out_h) MUMMU_H(1, 1, true);
        else MUMMU_H(1, 1, false);
    } else if (tile_rows == 16) {
        if (out_h)
            launch_kernel(grouped_gemm_q4k_f16_m16_kernel<GATE_UP, true>, grid, dim3(512), 0, s, w0, w1, a_in, sorted, k_slots, tiles,
                          n_tiles, in_dim, out_dim, act_h, act_q, y_out);
        else
            launch_kernel(grouped_gemm_q4k_f16_m16_kernel<GATE_UP, false>, grid, dim3(512), 0, s, w0, w1, a_in, sorted, k_slots, tiles,
                          n_tiles, in_dim, out_dim, act_h, act_q, y_out);
    } else {
        return hipErrorInvalidValue;
    }
#undef MUMMU_H
    return hipGetLastError();
}

template <bool GATE_UP>
static hipError_t launch_gemm_f32(const uint8_t *w0, const uint8_t *w1, const float *a_in, const int32_t *sorted, int k_slots,
                                  const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, int in_dim,
                                  int out_dim, float *act_out, float *y_out, hipStream_t s) {
    dim3 block(256), grid((unsigned)((max_tiles + 7) / 8 * 8) * (unsigned)((out_dim + kBN - 1) / kBN));
    if (tile_rows == 64)
        launch_kernel(grouped_gemm_f32_kernel<GATE_UP, 2>, grid, block, 0, s, w0, w1, a_in, sorted, k_slots, tiles, n_tiles, in_dim,
                      out_dim, act_out, y_out);
    else if (tile_rows == 32)
        launch_kernel(grouped_gemm_f32_kernel<GATE_UP, 1>, grid, block, 0, s, w0, w1, a_in, sorted, k_slots, tiles, n_tiles, in_dim,
                      out_dim, act_out, y_out);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

template <bool GATE_UP, int WT>
static hipError_t launch_gemm_f16(const uint8_t *w0, const uint8_t *w1, const _Float16 *act_in,
                                  const int32_t *sorted, int k_slots, const int32_t *tiles, const int32_t *n_tiles,
                                  int max_tiles, int tile_rows, int in_dim, int out_dim, _Float16 *act_out, float *y_out,
                                  hipStream_t s) {
    dim3 block(256), grid((unsigned)((max_tiles + 7) / 8 * 8) * (unsigned)((out_dim + kBN - 1) / kBN));
#define MUMMU_F16(MT)                                                                                                    \
    launch_kernel(grouped_gemm_f16_kernel<GATE_UP, MT, WT>, grid, block, 0, s, w0, w1, act_in, sorted, k_slots, tiles, n_tiles, \
                  in_dim, out_dim, act_out, y_out)
    switch (tile_rows) {
    case 32: MUMMU_F16(1); break;
    case 64: MUMMU_F16(2); break;
    case 96: MUMMU_F16(3); break;
    case 128: MUMMU_F16(4); break;
    default: return hipErrorInvalidValue;
    }
#undef MUMMU_F16
    return hipGetLastError();
}

hipError_t launch_gemm_gate_up(const ExpertBanks &b, const float *x, QAct64 xq, HAct xh, const int32_t *sorted, int k_slots,
                               const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, void *act16,
                               float *act32, QAct64 actq, HAct acth, hipStream_t s, bool q8_half) {
    if (!grouped_gemm_supported(b)) return hipErrorInvalidValue;
    if (q8_half) {
        // (x as halfs in xh.hi alone, as for the f16 banks)
        if (!grouped_gemm_q8_f16(b) || xh.hi == nullptr || xh.lo != nullptr) return hipErrorInvalidValue;
        return launch_gemm_f16<true, T_Q8_0>(b.gate, b.up, xh.hi, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, b.hidden,
                                             b.inter, (_Float16 *)act16, nullptr, s);
    }
    if (xh.hi != nullptr && xh.lo != nullptr) {
        if (!grouped_gemm_q4k_f16(b)) return hipErrorInvalidValue;
        const bool out_h = acth.hi != nullptr;
        if (out_h && !grouped_gemm_q4k_f16_down(b)) return hipErrorInvalidValue;
        return launch_gemm_q4k_f16<true>(b.gate, b.up, xh, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, b.hidden, b.inter,
                                         acth, actq, out_h, nullptr, s);
    }
    if (b.gate_type == T_F32)
        return launch_gemm_f32<true>(b.gate, b.up, x, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, b.hidden, b.inter, act32,
                                     nullptr, s);
    // (f16 and bf16 banks read x as halfs: xh.hi alone, from launch_convert_rows_f16)
    if ((b.gate_type == T_F16 || b.gate_type == T_BF16) && xh.hi == nullptr) return hipErrorInvalidValue;
    if (b.gate_type == T_F16)
        return launch_gemm_f16<true, T_F16>(b.gate, b.up, xh.hi, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, b.hidden,
                                            b.inter, (_Float16 *)act16, nullptr, s);
    if (b.gate_type == T_BF16)
        return launch_gemm_f16<true, T_BF16>(b.gate, b.up, xh.hi, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, b.hidden,
                                           b.inter, (_Float16 *)act16, nullptr, s);
    switch (b.gate_type) {
#define MUMMU_GU(T)                                                                                                          \
    case T:                                                                                                                  \
        return launch_gemm_q<T, true>(b.gate, b.up, xq, sorted, k_slots, tiles, n_tiles, max_tiles, tile_rows, true, b.hidden, b.inter, \
                                      actq, nullptr, s)
        MUMMU_GU(T_Q8_0);
        MUMMU_GU(T_Q4_K);
        MUMMU_GU(T_Q4_0);
        MUMMU_GU(T_Q4_1);
        MUMMU_GU(T_Q5_0);
        MUMMU_GU(T_Q5_1);
        MUMMU_GU(T_Q5_K);
        MUMMU_GU(T_Q6_K);
#undef MUMMU_GU
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm_down(const ExpertBanks &b, const void *act16, const float *act32, QAct64 actq, HAct acth, int n_assign,
                            const int32_t *tiles, const int32_t *n_tiles, int max_tiles, int tile_rows, float *y, hipStream_t s,
                            bool q8_half) {
    if (!grouped_gemm_supported(b)) return hipErrorInvalidValue;
    if (q8_half) {
        if (!grouped_gemm_q8_f16(b) || acth.hi != nullptr) return hipErrorInvalidValue;
        return launch_gemm_f16<false, T_Q8_0>(b.down, nullptr, (const _Float16 *)act16, nullptr, 1, tiles, n_tiles, max_tiles,
                                              tile_rows, b.inter, b.hidden, nullptr, y, s);
    }
    if (acth.hi != nullptr) {
        if (!grouped_gemm_q4k_f16_down(b)) return hipErrorInvalidValue;
        return launch_gemm_q4k_f16<false>(b.down, nullptr, acth, nullptr, 1, tiles, n_tiles, max_tiles, tile_rows, b.inter, b.hidden,
                                          HAct(), QAct64(), false, y, s);
    }
    if (b.down_type == T_F32)
        return launch_gemm_f32<false>(b.down, nullptr, act32, nullptr, 1, tiles, n_tiles, max_tiles, tile_rows, b.inter, b.hidden,
                                      nullptr, y, s);
    const bool few_rows = n_assign <= 64 * b.n_experts;  // an expert's rows fit one tile, on average
    if (b.down_type == T_F16)
        return launch_gemm_f16<false, T_F16>(b.down, nullptr, (const _Float16 *)act16, nullptr, 1, tiles, n_tiles, max_tiles,
                                             tile_rows, b.inter, b.hidden, nullptr, y, s);
    if (b.down_type == T_BF16)
        return launch_gemm_f16<false, T_BF16>(b.down, nullptr, (const _Float16 *)act16, nullptr, 1, tiles, n_tiles, max_tiles,
                                            tile_rows, b.inter, b.hidden, nullptr, y, s);
    switch (b.down_type) {
#define MUMMU_DN(T)                                                                                                      \
    case T:                                                                                                              \
        return launch_gemm_q<T, false>(b.down, nullptr, actq, nullptr, 1, tiles, n_tiles, max_tiles, tile_rows, few_rows, b.inter, b.hidden, \
                                       QAct64(), y, s)
        MUMMU_DN(T_Q8_0);
        MUMMU_DN(T_Q4_K);
        MUMMU_DN(T_Q4_0);
        MUMMU_DN(T_Q4_1);
        MUMMU_DN(T_Q5_0);
        MUMMU_DN(T_Q5_1);
        MUMMU_DN(T_Q5_K);
        MUMMU_DN(T_Q6_K);
#undef MUMMU_DN
    default: return hipErrorInvalidValue;
    }
}

}  // namespace mummu
