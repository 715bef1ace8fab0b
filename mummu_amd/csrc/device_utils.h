// Device-side helpers shared by the MoE kernels (gfx950, wave64).
//
// All translation units are compiled with -ffp-contract=off: a fused multiply-add happens
// only where the code writes fmaf/__builtin_fmaf, so "two roundings" stays two roundings.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mummu {

constexpr int kWave = 64;

// ggml tensor type ids (the values stored in GGUF tensor tables).
enum : int { T_F32 = 0, T_F16 = 1, T_Q8_0 = 8, T_Q4_K = 12, T_BF16 = 30 };

__host__ __device__ inline int block_elems(int t) {
    switch (t) {
    case T_F32: case T_F16: case T_BF16: return 1;
    case T_Q8_0: return 32;
    case T_Q4_K: return 256;
    default: return 0;
    }
}

__host__ __device__ inline int block_bytes(int t) {
    switch (t) {
    case T_F32: return 4;
    case T_F16: case T_BF16: return 2;
    case T_Q8_0: return 34;
    case T_Q4_K: return 144;
    default: return 0;
    }
}

// IEEE half bits -> f32, exact (subnormals included: gfx9 keeps f16 denormals).
__device__ inline float half_bits_to_float(uint16_t bits) {
    _Float16 h;
    __builtin_memcpy(&h, &bits, 2);
    return (float)h;
}

__device__ inline float bf16_bits_to_float(uint16_t bits) { return __uint_as_float((uint32_t)bits << 16); }

// Single-precision exp, specified operation by operation so the CPU checker can follow it
// bit for bit: magic-constant rounding of x*log2(e), Cody-Waite reduction, degree-5 Horner
// in fma form, exact two-step power-of-two scaling (subnormal results round once).
__device__ inline float det_expf(float x) {
    if (x != x) return x;
    if (x >= 88.7228394f) return __builtin_inff();
    if (x < -103.9720840f) return 0.0f;
    const float LOG2E = 1.44269502f;
    const float LN2_HI = 0.693359375f;
    const float LN2_LO = -2.12194440e-4f;
    const float MAGIC = 12582912.0f;
    float t = __builtin_fmaf(x, LOG2E, MAGIC);
    float n = __fsub_rn(t, MAGIC);
    float r = __builtin_fmaf(-n, LN2_HI, x);
    r = __builtin_fmaf(-n, LN2_LO, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float r2 = __fmul_rn(r, r);
    float y = __builtin_fmaf(p, r2, r);
    y = __fadd_rn(y, 1.0f);
    int ni = (int)n;
    int a = ni / 2;
    int b = ni - a;
    float sa = __uint_as_float((uint32_t)(a + 127) << 23);
    float sb = __uint_as_float((uint32_t)(b + 127) << 23);
    y = __fmul_rn(y, sa);
    y = __fmul_rn(y, sb);
    return y;
}

// x / (1 + e^-x), the ggml form: very negative x gives a clean -0.0.
__device__ inline float det_silu(float x) {
    float e = det_expf(-x);
    float den = __fadd_rn(1.0f, e);
    return __fdiv_rn(x, den);
}

// Butterfly sum over the whole wave, offsets 32,16,...,1.  Lane l ends with the value a
// halving tree (s[l] += s[l+off] for l < off) leaves in s[0]; addition commutes, so every
// lane holds the same bits.
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, kWave));
    return v;
}

// Butterfly sum over aligned groups of `width` lanes (width a power of two <= 64).
__device__ inline float group_sum(float v, int width) {
    for (int off = width >> 1; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

}  // namespace mummu
