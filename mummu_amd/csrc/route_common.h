// Device pieces shared by the router kernels: router weight loads and the one-wave softmax /
// top-k / renormalise of one token.
#pragma once

#include "device_utils.h"
#include "kernels.h"

namespace mummu {

constexpr int kMaxExpertsPerLane = 8;  // num_experts <= 512

template <int WT>
__device__ inline float load_w(const void *w, size_t i) {
    if constexpr (WT == T_F32) return ((const float *)w)[i];
    else if constexpr (WT == T_F16) return half_bits_to_float(((const uint16_t *)w)[i]);
    else return bf16_bits_to_float(((const uint16_t *)w)[i]);
}

// 8 consecutive weights starting at element i (i % 8 == 0, 16-byte aligned rows).
template <int WT>
__device__ inline void load_w8(const void *w, size_t i, float (&o)[8]) {
    if constexpr (WT == T_F32) {
        const float4 *p = (const float4 *)((const float *)w + i);
        float4 a = p[0], b = p[1];
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    } else {
        uint4 v = *(const uint4 *)((const uint16_t *)w + i);
        uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint16_t lo = (uint16_t)(u[j] & 0xFFFFu), hi = (uint16_t)(u[j] >> 16);
            if constexpr (WT == T_F16) {
                o[2 * j] = half_bits_to_float(lo);
                o[2 * j + 1] = half_bits_to_float(hi);
            } else {
                o[2 * j] = bf16_bits_to_float(lo);
                o[2 * j + 1] = bf16_bits_to_float(hi);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// One token's activation row held by one wave in the router's layout: lane l owns elements 8l .. 8l+7 of
// every 512-element chunk (hidden <= 512 * kWaveRowChunks, hidden % 8 == 0, 16-byte aligned rows).  Every load
// of the row goes out at once.  Lanes whose slice lies past the row's end re-read its first elements and never
// use them.
// ---------------------------------------------------------------------------------------
constexpr int kWaveRowChunks = 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));  // (a first-class vector type: arrays of it stay in registers)

struct WaveRow {
    f32x4 a[kWaveRowChunks], b[kWaveRowChunks];
};

__device__ __forceinline__ void wave_row_load(const float *__restrict__ xr, int hidden, int lane, WaveRow &r) {
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        const int base = lane * 8 + 512 * c;
        const int at = base < hidden ? base : 0;
        r.a[c] = ((const f32x4 *)(xr + at))[0];
        r.b[c] = ((const f32x4 *)(xr + at))[1];
    }
}

// 1 / sqrt(mean(x^2) + eps): the sum of squares as 512 strided partials (element i -> partial i mod 512, fused
// multiply-adds in ascending i), each lane's eight folded ((a0+a4)+(a1+a5))+((a2+a6)+(a3+a7)), then the pairwise
// tree over the lanes - the order the RmsNorm kernel and the router kernel use.  Every lane gets the result.
__device__ __forceinline__ float wave_row_rms_scale(const WaveRow &r, int hidden, int lane, float eps) {
    float a2[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        if (lane * 8 + 512 * c >= hidden) continue;
        const float xv[8] = {r.a[c].x, r.a[c].y, r.a[c].z, r.a[c].w, r.b[c].x, r.b[c].y, r.b[c].z, r.b[c].w};
#pragma unroll
        for (int j = 0; j < 8; j++) a2[j] = __builtin_fmaf(xv[j], xv[j], a2[j]);
    }
    float ss = __fadd_rn(__fadd_rn(__fadd_rn(a2[0], a2[4]), __fadd_rn(a2[1], a2[5])),
                         __fadd_rn(__fadd_rn(a2[2], a2[6]), __fadd_rn(a2[3], a2[7])));
    ss = wave_sum(ss);
    return __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ss, (float)hidden), eps)));
}

// x <- (x * rs) * gamma, two roundings per element.
__device__ __forceinline__ void wave_row_normalise(WaveRow &r, float rs, const float *__restrict__ gamma, int hidden, int lane) {
    f32x4 ga[kWaveRowChunks], gb[kWaveRowChunks];
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        const int base = lane * 8 + 512 * c;
        const int at = base < hidden ? base : 0;
        ga[c] = ((const f32x4 *)(gamma + at))[0];
        gb[c] = ((const f32x4 *)(gamma + at))[1];
    }
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        r.a[c].x = __fmul_rn(__fmul_rn(r.a[c].x, rs), ga[c].x);
        r.a[c].y = __fmul_rn(__fmul_rn(r.a[c].y, rs), ga[c].y);
        r.a[c].z = __fmul_rn(__fmul_rn(r.a[c].z, rs), ga[c].z);
        r.a[c].w = __fmul_rn(__fmul_rn(r.a[c].w, rs), ga[c].w);
        r.b[c].x = __fmul_rn(__fmul_rn(r.b[c].x, rs), gb[c].x);
        r.b[c].y = __fmul_rn(__fmul_rn(r.b[c].y, rs), gb[c].y);
        r.b[c].z = __fmul_rn(__fmul_rn(r.b[c].z, rs), gb[c].z);
        r.b[c].w = __fmul_rn(__fmul_rn(r.b[c].w, rs), gb[c].w);
    }
}

// A router row's weights in the same layout (all loads at once) ...
struct WaveRouterRow {
    float w[kWaveRowChunks][8];
};

template <int WT>
__device__ __forceinline__ void wave_router_row_load(const void *__restrict__ w, size_t wrow, int hidden, int lane, WaveRouterRow &r) {
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        const int base = lane * 8 + 512 * c;
        load_w8<WT>(w, wrow + (size_t)(base < hidden ? base : 0), r.w[c]);
    }
}

// ... and the logit <x, w> in the router's fixed order (the file comment of router.hip): every lane gets it.
__device__ __forceinline__ float wave_router_dot(const WaveRow &x, const WaveRouterRow &wr, int hidden, int lane) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < kWaveRowChunks; c++) {
        if (lane * 8 + 512 * c >= hidden) continue;  // (never adds: keeps -0 partials impossible either way)
        const float xv[8] = {x.a[c].x, x.a[c].y, x.a[c].z, x.a[c].w, x.b[c].x, x.b[c].y, x.b[c].z, x.b[c].w};
#pragma unroll
        for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(xv[j], wr.w[c][j], acc[j]);
    }
    const float s = __fadd_rn(__fadd_rn(__fadd_rn(acc[0], acc[4]), __fadd_rn(acc[1], acc[5])),
                              __fadd_rn(__fadd_rn(acc[2], acc[6]), __fadd_rn(acc[3], acc[7])));
    return wave_sum(s);
}

// ---------------------------------------------------------------------------------------
// softmax -> top-k -> renormalise, one wave per token.  Lane l holds experts l, l+64, ...
// Ties: strictly-greater wins, so the lower expert id keeps a tie and equal slots ascend
// by id (experts.rs:557-573; the stable descending sort of nn/moe.rs:2143-2144).
//
// The sequential sums and the ranking read every expert's value; the wave parks them in LDS
// and every lane streams them back with broadcast 16-byte reads, which keeps the serial
// chains to one add (or one compare) per element instead of a cross-lane move per element.
// ---------------------------------------------------------------------------------------
__device__ inline void wave_lds_sync() {
    // LDS traffic of one wave is issued in order; this only stops the compiler from moving
    // the reads above the writes.
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Per-wave LDS scratch of the router.
template <int JN>
struct RouteScratch {
    float p[64 * JN];   // per-expert values, expert order
    float w[64 * JN];   // selected probabilities, slot order
    int id[64 * JN];    // selected expert ids, slot order
};

// One wave routes one token whose logits sit in l[j] (expert lane + 64*j).  JN = experts held
// per lane (num_experts <= 64 * JN).  ANY_K = false leaves out the ranking path of k > 16 (the
// caller guarantees k <= 16), which is most of the code and of the registers.
template <int JN, bool ANY_K = true>
__device__ __forceinline__ void route_token(float (&l)[JN], int t, int n_experts, int k, int flavour, int norm,
                                   int32_t *__restrict__ ids, float *__restrict__ weights,
                                   unsigned long long *__restrict__ hits, int32_t *__restrict__ flags,
                                   RouteScratch<JN> &sc, int out_row = -1) {
    const int lane = threadIdx.x & 63;
    const size_t orow = out_row < 0 ? (size_t)t : (size_t)out_row;  // row of ids / weights this token's routing goes to
    float p[JN];
    bool bad = false;
    float mx = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < JN; j++) {
        const int e = lane + 64 * j;
        if (e < n_experts) {
            if (!(fabsf(l[j]) <= 3.402823466e38f)) {  // inf or NaN
                bad = true;
                atomicMin(&flags[FLAG_NONFINITE_INDEX], t * n_experts + e);
            }
            mx = fmaxf(mx, l[j]);
        }
    }
    if (__any(bad)) {
        // Refused like experts.rs:546-553: flag it and emit a harmless, in-range routing so
        // the kernels downstream stay inside their buffers; the host reports the error.
        if (lane == 0) atomicAdd(&flags[FLAG_NONFINITE], 1);
        for (int s = lane; s < k; s += 64) {
            ids[orow * k + s] = s;
            weights[orow * k + s] = 0.0f;
        }
        return;
    }
    mx = wave_max(mx);
    // experts past n_experts hold +0: it leaves a running sum unchanged bit for bit and never
    // outranks a real expert (not greater; on a tie at 0 its id is higher)
#pragma unroll
    for (int j = 0; j < JN; j++) {
        p[j] = (lane + 64 * j < n_experts) ? det_expf(__fsub_rn(l[j], mx)) : 0.0f;
        sc.p[lane + 64 * j] = p[j];
    }
    wave_lds_sync();

    // normaliser: sequential over ascending expert id (every lane computes the same sum); the
    // slots past n_experts hold +0 and are skipped in whole chunks of four
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
        // The f64 sum of at most 512 values in [0, 1] is EXACT, whatever the order, when every
        // non-zero value is at least 2^-20: such an f32 is a multiple of 2^-43, and a sum of those
        // that stays <= 2^9 fits f64's 53 bits.  Then a tree over the lanes gives the bits of the
        // sequential sum; otherwise (a probability below 2^-20) add in expert order as written.
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

    MUMMU_PHASE(12);
    if (JN == 1 && (!ANY_K || k <= 16)) {
        // one expert per lane: the rounds run on the bit patterns (a probability is a non-negative finite float, so it
        // orders like its bits; -1 marks a lane that is out of the running), and every lane remembers the slot it won
        // instead of lane 0 writing each round's winner
        // The renormaliser (the selected probabilities summed in slot order) builds up inside the rounds, where every
        // lane holds each round's maximum, so the winners write their own slot and nothing goes through LDS.
        int cand = lane < n_experts ? __float_as_int(p[0]) : -1;
        int my_slot = -1;
        float sum32 = 0.0f;
        double sum64 = 0.0;
        auto round = [&](int s) {
            const int best = wave_max_i32(cand);
            const int win = (int)__builtin_ctzll(__ballot(cand == best));  // lowest expert id holding the maximum
            my_slot = lane == win ? s : my_slot;
            cand = lane == win ? -1 : cand;
            const float bf = __int_as_float(best);
            sum32 = __fadd_rn(sum32, bf);
            sum64 = __dadd_rn(sum64, (double)bf);
        };
        if (k == 8) {  // the usual top-8 as straight-line code (a taken branch costs as much as half a round)
#pragma unroll
            for (int s = 0; s < 8; s++) round(s);
        } else {
            for (int s = 0; s < k; s++) round(s);
        }
        MUMMU_PHASE(13);
        float denom = 1.0f;
        if (flavour == 0) {
            if (norm) denom = sum32;
        } else {
            const float fs = (float)sum64;
            const float floor_v = 1.0f / 16384.0f;  // experts.rs:74
            denom = fs > floor_v ? fs : floor_v;
        }
        // (a lane past n_experts never wins a round while a real candidate is left: its -1 loses to every probability,
        // which is a finite non-negative float here - non-finite logits were refused above; the bound is kept all the same)
        if (my_slot >= 0 && lane < n_experts) {
            float wv = p[0];
            if (flavour != 0 || norm) wv = __fdiv_rn(wv, denom);
            ids[orow * k + my_slot] = lane;
            weights[orow * k + my_slot] = wv;
            if (hits) atomicAdd(&hits[lane], 1ULL);
        }
        return;
    } else if (!ANY_K || k <= 16) {
        // k rounds of "largest remaining probability, lowest id on a tie": the wave maximum,
        // then the first lane (and, within a lane, the first expert) that holds it
        float cand[JN];
#pragma unroll
        for (int j = 0; j < JN; j++) cand[j] = (lane + 64 * j < n_experts) ? p[j] : -1.0f;
        for (int s = 0; s < k; s++) {
            float best = cand[0];
#pragma unroll
            for (int j = 1; j < JN; j++) best = fmaxf(best, cand[j]);
            best = wave_max(best);
            // lowest expert id holding `best` (id = lane + 64*j)
            int my = 0x7FFFFFFF;
#pragma unroll
            for (int j = JN - 1; j >= 0; j--)
                if (cand[j] == best) my = lane + 64 * j;
            int win = my;
            const unsigned long long m = __ballot(my != 0x7FFFFFFF);
            if (JN == 1) {
                win = (int)__builtin_ctzll(m);
            } else if ((m & (m - 1)) == 0ull) {
                // one lane holds the maximum (the usual case): its lowest such expert wins
                win = __builtin_amdgcn_readlane(my, (int)__builtin_ctzll(m));
            } else {
                // minimum id over the wave
                float f = -(float)win;  // ids < 2^24: exact in f32, negated so that max finds the minimum
                f = wave_max(f);
                win = (int)(-f);
            }
#pragma unroll
            for (int j = 0; j < JN; j++)
                if (lane + 64 * j == win) cand[j] = -1.0f;
            if (lane == 0) {
                sc.w[s] = best;
                sc.id[s] = win;
            }
        }
    } else {
        // rank of each expert under (probability descending, id ascending); rank < k is its slot
        wave_lds_sync();
#pragma unroll
        for (int j = 0; j < JN; j++) sc.p[lane + 64 * j] = p[j];
        wave_lds_sync();
        int rank[JN];
#pragma unroll
        for (int j = 0; j < JN; j++) rank[j] = 0;
#pragma unroll
        for (int c = 0; c < 16 * JN; c++) {
            const float4 v = bp[c];
            const float q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int eq = 4 * c + i;
#pragma unroll
                for (int j = 0; j < JN; j++) rank[j] += (q[i] > p[j]) || (q[i] == p[j] && eq < lane + 64 * j);
            }
        }
#pragma unroll
        for (int j = 0; j < JN; j++) {
            if (lane + 64 * j < n_experts && rank[j] < k) {
                sc.w[rank[j]] = p[j];
                sc.id[rank[j]] = lane + 64 * j;
            }
        }
    }
    wave_lds_sync();
    MUMMU_PHASE(13);

    float denom = 1.0f;
    if (flavour == 0) {
        if (norm) {
            float d = 0.0f;
            for (int s = 0; s < k; s++) d = __fadd_rn(d, sc.w[s]);
            denom = d;
        }
    } else {
        double d = 0.0;
        for (int s = 0; s < k; s++) d = __dadd_rn(d, (double)sc.w[s]);
        const float fs = (float)d;
        const float floor_v = 1.0f / 16384.0f;  // experts.rs:74
        denom = fs > floor_v ? fs : floor_v;
    }
    const bool divide = flavour != 0 || norm;
    for (int s = lane; s < k; s += 64) {
        float wv = sc.w[s];
        const int id = sc.id[s];
        if (divide) wv = __fdiv_rn(wv, denom);
        ids[orow * k + s] = id;
        weights[orow * k + s] = wv;
        if (hits && (unsigned)id < (unsigned)n_experts) atomicAdd(&hits[id], 1ULL);
    }
}

}  // namespace mummu
