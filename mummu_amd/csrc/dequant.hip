// gguf::dequantize on the device, bit for bit (reference: crates/mummu/src/gguf.rs:1403-1463
// and the per-type functions :1426-1436 F32/F16/BF16, :1535-1543 Q8_0, :1547-1610 Q4_0 / Q4_1 /
// Q5_0 / Q5_1, :1685-1726 Q4_K, :1731-1765 Q5_K, :1769-1797 Q6_K).
//
// This kernel exists to prove that the bytes resident in HBM decode to exactly the f32
// weights the reference would compute; the expert-product kernels read the same bytes but
// never materialise f32 weights.  One thread per output element; every multiply and
// subtract is a separately rounded IEEE operation in the reference's grouping:
//   Q8_0:        d * q
//   Q4_0, Q5_0:  d * (q - 8), d * (q - 16)
//   Q4_1, Q5_1:  (d * q) + m
//   Q4_K, Q5_K:  (d * sc) * q  -  (dmin * m)
//   Q6_K:        (d * sc) * (q - 32)
#include "device_utils.h"
#include "kernels.h"

namespace mummu {

__device__ inline void q4k_scale_min(const uint8_t *s, int j, float &sc, float &mn) {
    // ggml get_scale_min_k4 (gguf.rs:1685-1697)
    uint32_t a, b;
    if (j < 4) {
        a = s[j] & 63u;
        b = s[j + 4] & 63u;
    } else {
        a = (s[j + 4] & 0x0Fu) | ((uint32_t)(s[j - 4] >> 6) << 4);
        b = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
    sc = (float)a;
    mn = (float)b;
}

template <int TYPE>
__global__ void dequantize_kernel(const uint8_t *__restrict__ bytes, size_t n_elems, float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_elems) return;
    if constexpr (TYPE == T_F32) {
        const uint8_t *p = bytes + i * 4;
        uint32_t b = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
        out[i] = __uint_as_float(b);
    } else if constexpr (TYPE == T_F16) {
        const uint8_t *p = bytes + i * 2;
        out[i] = half_bits_to_float((uint16_t)(p[0] | (p[1] << 8)));
    } else if constexpr (TYPE == T_BF16) {
        const uint8_t *p = bytes + i * 2;
        out[i] = bf16_bits_to_float((uint16_t)(p[0] | (p[1] << 8)));
    } else if constexpr (TYPE == T_Q8_0) {
        const uint8_t *blk = bytes + (i / 32) * 34;
        float d = half_bits_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
        out[i] = __fmul_rn(d, (float)(int8_t)blk[2 + (i % 32)]);
    } else if constexpr (TYPE == T_Q4_K) {
        const uint8_t *blk = bytes + (i / 256) * 144;
        int within = (int)(i % 256);
        int sub = within / 32;          // sub-block 0..7: chunk = sub/2, low nibbles first
        int pos = within % 32;
        float d = half_bits_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
        float dmin = half_bits_to_float((uint16_t)(blk[2] | (blk[3] << 8)));
        float sc, mn;
        q4k_scale_min(blk + 4, sub, sc, mn);
        uint8_t byte = blk[16 + (sub / 2) * 32 + pos];
        uint32_t q = (sub & 1) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0F);
        float product = __fmul_rn(__fmul_rn(d, sc), (float)q);
        out[i] = __fsub_rn(product, __fmul_rn(dmin, mn));
    } else if constexpr (TYPE == T_Q4_0 || TYPE == T_Q4_1 || TYPE == T_Q5_0 || TYPE == T_Q5_1) {
        // 32-element blocks: f16 d (, f16 m) (, u32 fifth bits), 16 bytes of nibbles; byte j holds
        // element j in its low nibble and element j+16 in its high nibble
        constexpr bool has_m = TYPE == T_Q4_1 || TYPE == T_Q5_1;
        constexpr bool has_h = TYPE == T_Q5_0 || TYPE == T_Q5_1;
        const uint8_t *blk = bytes + (i / 32) * (size_t)block_bytes(TYPE);
        const int pos = (int)(i % 32), j = pos & 15, hi = pos >> 4;
        const float d = half_bits_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
        const uint8_t *p = blk + 2;
        float m = 0.0f;
        if constexpr (has_m) {
            m = half_bits_to_float((uint16_t)(p[0] | (p[1] << 8)));
            p += 2;
        }
        int q;
        if constexpr (has_h) {
            const uint32_t qh = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
            p += 4;
            q = (int)(hi ? p[j] >> 4 : p[j] & 0x0F) | (int)(((qh >> pos) & 1u) << 4);
        } else {
            q = (int)(hi ? p[j] >> 4 : p[j] & 0x0F);
        }
        if constexpr (has_m) out[i] = __fadd_rn(__fmul_rn(d, (float)q), m);
        else out[i] = __fmul_rn(d, (float)(q - (has_h ? 16 : 8)));
    } else if constexpr (TYPE == T_Q5_K) {
        const uint8_t *blk = bytes + (i / 256) * 176;
        const int within = (int)(i % 256), sub = within / 32, pos = within % 32;
        const float d = half_bits_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
        const float dmin = half_bits_to_float((uint16_t)(blk[2] | (blk[3] << 8)));
        float sc, mn;
        q4k_scale_min(blk + 4, sub, sc, mn);
        const uint8_t byte = blk[48 + (sub / 2) * 32 + pos];
        const int fifth = (blk[16 + pos] >> sub) & 1;  // bit 2*chunk for low nibbles, 2*chunk+1 for high
        const int q = (int)((sub & 1) ? (byte >> 4) : (byte & 0x0F)) + 16 * fifth;
        const float product = __fmul_rn(__fmul_rn(d, sc), (float)q);
        out[i] = __fsub_rn(product, __fmul_rn(dmin, mn));
    } else if constexpr (TYPE == T_Q6_K) {
        const uint8_t *blk = bytes + (i / 256) * 210;
        const int within = (int)(i % 256), half = within / 128, r = within % 128, grp = r / 32, l = r % 32;
        const uint8_t lo = blk[half * 64 + (grp & 1) * 32 + l];
        const uint8_t hb = blk[128 + half * 32 + l];
        const int q = (int)((grp < 2 ? lo & 0x0F : lo >> 4) | (((hb >> (2 * grp)) & 3) << 4)) - 32;
        const float sc = (float)(int8_t)blk[192 + half * 8 + 2 * grp + l / 16];
        const float d = half_bits_to_float((uint16_t)(blk[208] | (blk[209] << 8)));
        out[i] = __fmul_rn(__fmul_rn(d, sc), (float)q);
    }
}

hipError_t launch_dequantize(int type, const uint8_t *bytes, size_t nblocks, float *out, hipStream_t s) {
    size_t n = nblocks * (size_t)block_elems(type);
    if (n == 0) return hipSuccess;
    dim3 block(256), grid((unsigned)((n + 255) / 256));
    switch (type) {
    case T_F32: launch_kernel(dequantize_kernel<T_F32>, grid, block, 0, s, bytes, n, out); break;
    case T_F16: launch_kernel(dequantize_kernel<T_F16>, grid, block, 0, s, bytes, n, out); break;
    case T_BF16: launch_kernel(dequantize_kernel<T_BF16>, grid, block, 0, s, bytes, n, out); break;
    case T_Q8_0: launch_kernel(dequantize_kernel<T_Q8_0>, grid, block, 0, s, bytes, n, out); break;
    case T_Q4_K: launch_kernel(dequantize_kernel<T_Q4_K>, grid, block, 0, s, bytes, n, out); break;
    case T_Q4_0: launch_kernel(dequantize_kernel<T_Q4_0>, grid, block, 0, s, bytes, n, out); break;
    case T_Q4_1: launch_kernel(dequantize_kernel<T_Q4_1>, grid, block, 0, s, bytes, n, out); break;
    case T_Q5_0: launch_kernel(dequantize_kernel<T_Q5_0>, grid, block, 0, s, bytes, n, out); break;
    case T_Q5_1: launch_kernel(dequantize_kernel<T_Q5_1>, grid, block, 0, s, bytes, n, out); break;
    case T_Q5_K: launch_kernel(dequantize_kernel<T_Q5_K>, grid, block, 0, s, bytes, n, out); break;
    case T_Q6_K: launch_kernel(dequantize_kernel<T_Q6_K>, grid, block, 0, s, bytes, n, out); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace mummu
