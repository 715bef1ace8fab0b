// 16-bit block-scaled activations for the integer expert products.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"

namespace mummu {

// A matrix of activations quantized for the integer expert products: rows x D elements,
// 16-bit values xq = 256*hi + lo with one f32 scale and one integer sum per 16 elements.
//   hi, lo : int8  [rows][D]        scale : f32 [rows][D/16]       sum : int32 [rows][D/16]
struct QAct {
    int8_t *hi = nullptr;
    int8_t *lo = nullptr;
    float *scale = nullptr;
    int32_t *sum = nullptr;
};

// Quantize 16 consecutive activations held one per lane in an aligned 16-lane row (an inactive
// row holds zeros): every lane gets its hi/lo bytes and the block's scale and integer sum.
__device__ inline void quantize16(float v, int &hi, int &lo, float &scale, int &sum) {
    float m = fabsf(v);
    m = fmaxf(m, dpp_move<0xB1>(m));
    m = fmaxf(m, dpp_move<0x4E>(m));
    m = fmaxf(m, dpp_move<0x141>(m));
    m = fmaxf(m, dpp_move<0x140>(m));
    const float inv = m > 0.0f ? __fdiv_rn(32512.0f, m) : 0.0f;
    int xq = (int)__builtin_rintf(__fmul_rn(v, inv));
    xq = xq > 32512 ? 32512 : (xq < -32512 ? -32512 : xq);
    lo = ((xq + 128) & 255) - 128;
    hi = (xq - lo) >> 8;
    sum = xq;
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xF, 0xF, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x140, 0xF, 0xF, false);
    scale = m > 0.0f ? __fdiv_rn(m, 32512.0f) : 0.0f;
}

// ... and store them: the lanes write their hi/lo bytes, the lane of the block's first element
// the block scale and sum.
__device__ inline void quantize_store16(float v, bool active, const QAct &q, size_t row, int d, int elem) {
    int hi, lo, sum;
    float scale;
    quantize16(v, hi, lo, scale, sum);
    if (active) {
        q.hi[row * (size_t)d + elem] = (int8_t)hi;
        q.lo[row * (size_t)d + elem] = (int8_t)lo;
        if ((elem & 15) == 0) {
            q.scale[row * (size_t)(d / 16) + (elem >> 4)] = scale;
            q.sum[row * (size_t)(d / 16) + (elem >> 4)] = sum;
        }
    }
}

// Activations quantized for the batched integer products: the same 16-bit hi/lo planes, with one
// f32 scale per 64 elements and, per 32 elements, ssum = scale * (sum of the 16-bit values).
//   hi, lo : int8 [rows][D]       scale : f32 [rows][D/64]       ssum : f32 [rows][D/32]
struct QAct64 {
    int8_t *hi = nullptr;
    int8_t *lo = nullptr;
    float *scale = nullptr;
    float *ssum = nullptr;
};

// Quantize 64 consecutive activations held four per lane in an aligned 16-lane row (lane i holds
// elements 4i..4i+3; an inactive row holds zeros) and store them.  elem0 is the index of this
// lane's first element within the matrix row.
__device__ inline void quantize_store64(float4 v, bool active, const QAct64 &q, size_t row, int d, int elem0) {
    float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    m = fmaxf(m, dpp_move<0xB1>(m));
    m = fmaxf(m, dpp_move<0x4E>(m));
    m = fmaxf(m, dpp_move<0x141>(m));
    m = fmaxf(m, dpp_move<0x140>(m));
    const float inv = m > 0.0f ? __fdiv_rn(32512.0f, m) : 0.0f;
    const float scale = m > 0.0f ? __fdiv_rn(m, 32512.0f) : 0.0f;
    const float f[4] = {v.x, v.y, v.z, v.w};
    uint32_t hi_w = 0, lo_w = 0;
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int xq = (int)__builtin_rintf(__fmul_rn(f[i], inv));
        xq = xq > 32512 ? 32512 : (xq < -32512 ? -32512 : xq);
        const int lo = ((xq + 128) & 255) - 128;
        const int hi = (xq - lo) >> 8;
        hi_w |= (uint32_t)(hi & 255) << (8 * i);
        lo_w |= (uint32_t)(lo & 255) << (8 * i);
        sum += xq;
    }
    // 32 elements = 8 lanes
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, false);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xF, 0xF, false);
    if (active) {
        *(uint32_t *)(q.hi + row * (size_t)d + elem0) = hi_w;
        *(uint32_t *)(q.lo + row * (size_t)d + elem0) = lo_w;
        if ((elem0 & 31) == 0) q.ssum[row * (size_t)(d / 32) + (elem0 >> 5)] = __fmul_rn(scale, (float)sum);
        if ((elem0 & 63) == 0) q.scale[row * (size_t)(d / 64) + (elem0 >> 6)] = scale;
    }
}

// Activations for the products of Q4_K banks on the f16 matrix units: every element as a pair of
// halfs, x = scale * (hi + lo) with hi = f16(x / scale), lo = f16(x / scale - hi), and a power-of-two
// scale chosen so that the largest |x / scale| it covers lies in [2^9, 2^10): 22 significant bits per
// element (elements more than 2^24 below that largest one keep an absolute error of 2^-25 of it), and
// sums of 32 scaled elements stay below 2^15, inside a half's range.  The scale array has one entry per
// 128 elements; a producer that sees whole rows (quantize_rows_h) writes the same scale into all of a
// row's entries, one that sees 128 columns at a time (the gate/up epilogue) a scale per entry.
//   hi, lo : f16 [rows][D]      scale : f32 [rows][D/128]      ssum : f32 [rows][D/32], sum of x / scale
struct HAct {
    _Float16 *hi = nullptr;
    _Float16 *lo = nullptr;
    float *scale = nullptr;
    float *ssum = nullptr;
};

// The scale for a largest magnitude m = f * 2^ex, f in [0.5, 1): x / scale = x * 2^(10 - ex).
// A non-finite m (exponent 255) gives hi = inf and lo = inf - inf = NaN for an infinite element: a row that holds an
// infinity comes out NaN where the reference's f32 product gives an infinity (non-finite rows are outside what the
// parity tests pin).
__device__ inline void hact_scale_of(float m, float &inv, float &scale) {
    int ex = (int)((__float_as_uint(m) >> 23) & 255u) - 126;
    ex = ex < -116 ? -116 : ex;
    inv = __uint_as_float((uint32_t)(137 - ex) << 23);
    scale = __uint_as_float((uint32_t)(117 + ex) << 23);
}

// Store 128 consecutive activations held four per lane in an aligned 32-lane group (lane i holds
// elements 4i..4i+3; an inactive group holds zeros).  elem0: this lane's first element in the row.
// row_max < 0: the scale comes from these 128 elements; else from row_max, the largest magnitude of the row.
__device__ inline void hact_store128(float4 v, bool active, const HAct &q, size_t row, int d, int elem0, float row_max = -1.0f) {
    float m = row_max;
    if (row_max < 0.0f) {
        m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        m = fmaxf(m, dpp_move<0xB1>(m));
        m = fmaxf(m, dpp_move<0x4E>(m));
        m = fmaxf(m, dpp_move<0x141>(m));
        m = fmaxf(m, dpp_move<0x140>(m));
        m = fmaxf(m, __shfl_xor(m, 16, 64));
    }
    float inv, scale;
    hact_scale_of(m, inv, scale);
    const float f[4] = {__fmul_rn(v.x, inv), __fmul_rn(v.y, inv), __fmul_rn(v.z, inv), __fmul_rn(v.w, inv)};
    _Float16 hi[4], lo[4];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        hi[i] = (_Float16)f[i];
        lo[i] = (_Float16)__fsub_rn(f[i], (float)hi[i]);
        sum = __fadd_rn(sum, f[i]);
    }
    // 32 elements = 8 lanes
    sum = __fadd_rn(sum, dpp_move<0xB1>(sum));
    sum = __fadd_rn(sum, dpp_move<0x4E>(sum));
    sum = __fadd_rn(sum, dpp_move<0x141>(sum));
    if (active) {
        uint2 hw, lw;
        __builtin_memcpy(&hw, hi, 8);
        __builtin_memcpy(&lw, lo, 8);
        *(uint2 *)(q.hi + row * (size_t)d + elem0) = hw;
        *(uint2 *)(q.lo + row * (size_t)d + elem0) = lw;
        if ((elem0 & 31) == 0) q.ssum[row * (size_t)(d / 32) + (elem0 >> 5)] = sum;
        if ((elem0 & 127) == 0) q.scale[row * (size_t)(d / 128) + (elem0 >> 7)] = scale;
    }
}

// One workgroup of NT threads turns row `row` of x [n, d] into HAct with one scale for the whole row (d % 128 == 0):
// the row's largest magnitude first, then the row NT * 4 elements at a time.  s_max: NT / 64 floats of LDS.
template <int NT>
__device__ inline void hact_quantize_row(const float *__restrict__ x, int d, const HAct &q, int row, float *s_max) {
    const int tid = threadIdx.x;
    const float *xr = x + (size_t)row * (size_t)d;
    float m = 0.0f;
    for (int e0 = tid * 4; e0 < d; e0 += NT * 4) {
        const float4 v = *(const float4 *)(xr + e0);
        m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    m = wave_max(m);
    if ((tid & 63) == 0) s_max[tid >> 6] = m;
    __syncthreads();
    m = s_max[0];
#pragma unroll
    for (int w = 1; w < NT / 64; w++) m = fmaxf(m, s_max[w]);
    for (int e0 = tid * 4; e0 - tid * 4 < d; e0 += NT * 4) {   // (whole 32-lane groups run together: d is a multiple of 128)
        const bool active = e0 < d;
        const float4 v = active ? *(const float4 *)(xr + e0) : make_float4(0.f, 0.f, 0.f, 0.f);
        hact_store128(v, active, q, (size_t)row, d, e0, m);
    }
}

}  // namespace mummu
