// Device-side helpers shared by the MoE kernels (gfx950, wave64).
//
// All translation units are compiled with -ffp-contract=off: a fused multiply-add happens
// only where the code writes fmaf/__builtin_fmaf, so "two roundings" stays two roundings.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <type_traits>

namespace mummu {

// Every kernel of the library is launched through launch_kernel().  When the calling thread has
// set g_launch_timing (the per-kernel timing mode of the C ABI), the two events are bound to
// the dispatch itself and take its start and end timestamps - the duration a kernel trace
// reports - instead of bracketing it with marker packets; otherwise this is a plain launch.
struct LaunchTiming {
    hipEvent_t start = nullptr, stop = nullptr;
};
extern thread_local LaunchTiming g_launch_timing;

template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                          Args &&...args) {
    hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds_bytes, stream, g_launch_timing.start, g_launch_timing.stop, 0,
                          static_cast<KArgs>(args)...);
}


constexpr int kWave = 64;

// Phase marks for kernel timing studies.  A normal build compiles them away; with
// -DMUMMU_TRACE every wave stores the constant 100 MHz wall clock at each mark into a caller-provided buffer
// (16 slots per wave), set per translation unit through mummu_trace_set_<unit>(buffer, waves it holds).
#ifdef MUMMU_TRACE
static __device__ long long *g_trace_buf = nullptr;
static __device__ long long g_trace_waves = 0;  // waves the buffer has room for; a wave past it records nothing
#ifndef MUMMU_TRACE_MASK
#define MUMMU_TRACE_MASK 0xFFFF  // which of the 16 marks are compiled in (every mark costs a clock read and a store)
#endif
#define MUMMU_TRACE_WAVE ((long long)(blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6))
#define MUMMU_PHASE(ph)                                                                                           \
    do {                                                                                                          \
        if (((MUMMU_TRACE_MASK >> (ph)) & 1) && g_trace_buf && (threadIdx.x & 63) == 0 &&                         \
            MUMMU_TRACE_WAVE < g_trace_waves)                                                                     \
            g_trace_buf[MUMMU_TRACE_WAVE * 16 + (ph)] = wall_clock64();                                           \
    } while (0)
#define MUMMU_TRACE_UNIT(name)                                                                        \
    extern "C" __attribute__((visibility("default"))) int mummu_trace_set_##name(void *p, long long waves) { \
        if (hipMemcpyToSymbol(HIP_SYMBOL(mummu::g_trace_waves), &waves, sizeof(waves)) != hipSuccess) return 1; \
        return (int)hipMemcpyToSymbol(HIP_SYMBOL(mummu::g_trace_buf), &p, sizeof(p));                  \
    }
// Loop timers: MARK(i) adds the time since the previous mark to slot i; STORE writes the slot sums
// (slot 6 = first mark's clock, slot 7 = last) to the wave's 8 trace words.
#define MUMMU_TIMER_DECL long long tm_acc_[8] = {0, 0, 0, 0, 0, 0, 0, 0}, tm_last_ = wall_clock64(); tm_acc_[6] = tm_last_
#define MUMMU_TIMER_MARK(i)                      \
    do {                                         \
        const long long now_ = wall_clock64();   \
        tm_acc_[i] += now_ - tm_last_;           \
        tm_last_ = now_;                         \
    } while (0)
#define MUMMU_TIMER_STORE                                                                                         \
    do {                                                                                                          \
        tm_acc_[7] = tm_last_;                                                                                    \
        if (g_trace_buf && (threadIdx.x & 63) == 0 && MUMMU_TRACE_WAVE < g_trace_waves)                           \
            for (int i_ = 0; i_ < 8; i_++) g_trace_buf[MUMMU_TRACE_WAVE * 16 + i_] = tm_acc_[i_];                 \
    } while (0)
#else
#define MUMMU_PHASE(ph) do { } while (0)
#define MUMMU_TRACE_UNIT(name)
#define MUMMU_TIMER_DECL do { } while (0)
#define MUMMU_TIMER_MARK(i) do { } while (0)
#define MUMMU_TIMER_STORE do { } while (0)
#endif

// Keeps code on either side where it was written: the compiler may not move memory accesses
// across it (so a prefetch stays issued early instead of being sunk next to its first use) and
// the instruction scheduler may not move anything across it.  Emits no instruction and waits for
// nothing.
#define MUMMU_CODE_FENCE()                      \
    do {                                        \
        asm volatile("" ::: "memory");          \
        __builtin_amdgcn_sched_barrier(0);      \
    } while (0)

// ggml tensor type ids (the values stored in GGUF tensor tables).
enum : int {
    T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_0 = 8,
    T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14, T_BF16 = 30
};

__host__ __device__ constexpr int block_elems(int t) {
    switch (t) {
    case T_F32: case T_F16: case T_BF16: return 1;
    case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q8_0: return 32;
    case T_Q4_K: case T_Q5_K: case T_Q6_K: return 256;
    default: return 0;
    }
}

__host__ __device__ constexpr int block_bytes(int t) {
    switch (t) {
    case T_F32: return 4;
    case T_F16: case T_BF16: return 2;
    case T_Q4_0: return 18;
    case T_Q4_1: return 20;
    case T_Q5_0: return 22;
    case T_Q5_1: return 24;
    case T_Q8_0: return 34;
    case T_Q4_K: return 144;
    case T_Q5_K: return 176;
    case T_Q6_K: return 210;
    default: return 0;
    }
}

// The block-quantized types (everything but the plain float types).
__host__ __device__ constexpr bool is_quant_type(int t) { return block_elems(t) > 1; }

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

// Butterfly sum over aligned groups of `width` lanes (width a power of two <= 64).
__device__ inline float group_sum(float v, int width) {
    for (int off = width >> 1; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, kWave));
    return v;
}

// ---- cross-lane sums at VALU speed (DPP inside a 16-lane row, gfx950 lane swaps across rows) ----
template <int CTRL>
__device__ inline float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}

// Sum over aligned groups of WIDTH lanes inside a 16-lane row (WIDTH in {1,2,4,8,16}); every
// lane of a group ends with the group's sum.  Steps: xor 1, xor 2 (quad permutes), then the
// half-row and row mirrors, which pair lanes of the two already-uniform halves.
template <int WIDTH>
__device__ inline float row_group_sum(float v) {
    if constexpr (WIDTH >= 2) v = __fadd_rn(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    if constexpr (WIDTH >= 4) v = __fadd_rn(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    if constexpr (WIDTH >= 8) v = __fadd_rn(v, dpp_move<0x141>(v));  // row_half_mirror
    if constexpr (WIDTH >= 16) v = __fadd_rn(v, dpp_move<0x140>(v)); // row_mirror
    return v;
}

// v_permlane32_swap: lanes 0-31 receive a[l] + a[l+32], lanes 32-63 receive b[l-32] + b[l].
// With a == b this is the xor-32 butterfly step; with two values it also halves the work.
__device__ inline float swap32_add(float a, float b) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(a), __float_as_int(b), false, false);
    return __fadd_rn(__int_as_float(r[0]), __int_as_float(r[1]));
}

// v_permlane16_swap: even 16-lane rows receive a[row] + a[row+1], odd rows b[row-1] + b[row].
__device__ inline float swap16_add(float a, float b) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_int(a), __float_as_int(b), false, false);
    return __fadd_rn(__int_as_float(r[0]), __int_as_float(r[1]));
}

// Sum over the whole wave as the pairwise tree over adjacent lanes: butterfly offsets
// 1,2,4,8,16,32 (s[l] += s[l+off] for l a multiple of 2*off leaves the same value in s[0]).
// Addition commutes, so every lane ends with the same bits.  Offsets 1 and 2 are quad permutes,
// 4 and 8 the half-row and row mirrors (the mirrored partner holds the same value as the xor
// partner, because the smaller groups are already uniform), 16 and 32 the gfx950 lane swaps:
// no LDS round trip anywhere.  The whole wave must be active.
__device__ inline float wave_sum(float v) {
    v = row_group_sum<16>(v);
    v = swap16_add(v, v);
    return swap32_add(v, v);
}

// Number of finished sums a lane holds after reduce_partials<NV, GROUP>.
template <int NV, int GROUP>
__host__ __device__ constexpr int reduced_count() {
    if (GROUP == 64) return NV >= 4 ? NV / 4 : 1;
    if (GROUP == 32) return NV >= 2 ? NV / 2 : 1;
    return NV;
}

// Reduce NV per-lane partials, each over aligned groups of GROUP lanes (power of two), and
// leave reduced_count<NV, GROUP>() finished sums in v[0..count): the value with original index
// (returned offset) + j sits in v[j].  Crossing the 32- and 16-lane boundaries halves the number
// of values a lane carries (the two halves of the group finish different values), so those
// steps are shared between values.
template <int NV, int GROUP>
__device__ inline int reduce_partials(float (&v)[NV], int lane) {
    int offset = 0;
    if constexpr (GROUP == 64) {
        if constexpr (NV >= 4) {
#pragma unroll
            for (int j = 0; j < NV / 2; j++) v[j] = swap32_add(v[j], v[j + NV / 2]);
#pragma unroll
            for (int j = 0; j < NV / 4; j++) v[j] = swap16_add(v[j], v[j + NV / 4]);
            offset = ((lane >> 5) & 1) * (NV / 2) + ((lane >> 4) & 1) * (NV / 4);
        } else if constexpr (NV == 2) {
            v[0] = swap32_add(v[0], v[1]);
            v[0] = swap16_add(v[0], v[0]);
            offset = (lane >> 5) & 1;
        } else {
            v[0] = swap32_add(v[0], v[0]);
            v[0] = swap16_add(v[0], v[0]);
        }
    } else if constexpr (GROUP == 32) {
        if constexpr (NV >= 2) {
#pragma unroll
            for (int j = 0; j < NV / 2; j++) v[j] = swap16_add(v[j], v[j + NV / 2]);
            offset = ((lane >> 4) & 1) * (NV / 2);
        } else {
            v[0] = swap16_add(v[0], v[0]);
        }
    }
    constexpr int count = reduced_count<NV, GROUP>();
    constexpr int width = GROUP < 16 ? GROUP : 16;
#pragma unroll
    for (int j = 0; j < count; j++) v[j] = row_group_sum<width>(v[j]);
    return offset;
}

// Calls f(std::integral_constant<int, G>{}) with G the lane-group size g in {64, 32, ..., 1}.
template <typename F>
__device__ inline void dispatch_group(int g, F &&f) {
    switch (g) {
    case 64: f(std::integral_constant<int, 64>{}); break;
    case 32: f(std::integral_constant<int, 32>{}); break;
    case 16: f(std::integral_constant<int, 16>{}); break;
    case 8: f(std::integral_constant<int, 8>{}); break;
    case 4: f(std::integral_constant<int, 4>{}); break;
    case 2: f(std::integral_constant<int, 2>{}); break;
    default: f(std::integral_constant<int, 1>{}); break;
    }
}

// Maximum of a signed integer over the wave, every lane gets it.  The four steps inside a 16-lane row are single
// v_max_i32 instructions reading their first operand through DPP (written as such: left to itself the compiler makes a
// move and a maximum of each; the s_nop covers the two wait states a DPP read needs after a write of the same
// register), then the two lane swaps across rows.  Non-negative finite floats order like their bit patterns, so this
// also serves as their maximum.
__device__ inline int wave_max_i32(int v) {
    asm("s_nop 1\n\tv_max_i32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_i32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_i32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_i32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf"
        : "+v"(v));
    // (the swaps return unsigned words: compare them as the signed values they are)
    auto a = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    const int a0 = (int)a[0], a1 = (int)a[1];
    v = a0 > a1 ? a0 : a1;
    auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    const int b0 = (int)b[0], b1 = (int)b[1];
    return b0 > b1 ? b0 : b1;
}

// Maximum over the wave, every lane gets it: four DPP steps inside each 16-lane row, then the
// two lane swaps across rows.
__device__ inline float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_int(v), __float_as_int(v), false, false);
    v = fmaxf(__int_as_float(a[0]), __int_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_int(v), __float_as_int(v), false, false);
    return fmaxf(__int_as_float(b[0]), __int_as_float(b[1]));
}

}  // namespace mummu
