// Packed GEMV over burn's block-32 quantized weight layout: the custom-op seam of the reference,
// Q4GemvOps::q4s_gemv (nn/packed_gemv.rs:248-260), whose CubeCL kernel is packed_gemv_kernel
// (nn/packed_gemv.rs:370-451).
//
// Layout (nn/packed_gemv.rs:26-29, pack.rs:940-985): the weight is [K, N] row-major, values two's
// complement in 4 (Q4S) or 8 (Q8S) bits, element j of a u32 word at bits j*bits, words running along
// N; one f32 scale per (k, block of 32 consecutive n).  The op is
//     y[n] = sum_k float(q(k, n)) * (x[k] * scale(k, n / 32)),
// the product x*scale rounded, the product with q rounded, then added (two roundings, as the
// reference's kernel and its dequantize-then-matmul form do).
//
// Mapping: a thread owns one word column (8 or 4 outputs) and walks a slice of K, so at any k the
// 64 lanes of a wave read 64 consecutive words; the four waves of a workgroup and gridDim.y
// workgroups split K (a decode-shape weight has too few word columns to fill 256 CUs otherwise).
// The slices of a workgroup meet in LDS and are added in ascending order, the workgroups' partials
// by a second small kernel in ascending order: the result does not depend on timing.  Up to 64
// rows of x go in one launch, one, two or four to a thread (blockIdx.z = the group), where the
// reference runs a short prefill row by row through the same op (nn/packed_gemv.rs:138-150); a row's
// sums are the same whatever shares the launch.
#include "device_utils.h"
#include "kernels.h"

#include <mutex>
#include <string>

#include "../../include/mummu_moe.h"

MUMMU_TRACE_UNIT(packed_gemv)

namespace mummu {

constexpr int kPgWaves = 4;

// R rows of x per thread (blockIdx.z = group of R rows): a word is loaded and decoded once for all of them.
// kPgUnroll K steps are loaded before the first is used, so a thread keeps that many words in flight.
constexpr int kPgUnroll = 16;

template <int BITS, int R>
__global__ __launch_bounds__(64 * kPgWaves) void packed_gemv_kernel(const uint32_t *__restrict__ words,
                                                                    const float *__restrict__ scales,
                                                                    const float *__restrict__ x, int m, int k_len, int n_words,
                                                                    int n_blocks, int k_chunk, float *__restrict__ out,
                                                                    size_t out_slice_stride) {
    constexpr int PER = 32 / BITS;
    __shared__ float s_part[kPgWaves][R][64][PER + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wc = blockIdx.x * 64 + lane;
    const bool valid = wc < n_words;
    const int row0 = blockIdx.z * R;
    const float *xr[R];
#pragma unroll
    for (int r = 0; r < R; r++) xr[r] = x + (size_t)(row0 + r < m ? row0 + r : m - 1) * (size_t)k_len;  // (past m: computed, not stored)
    const int slice = blockIdx.y * kPgWaves + wave;
    const int k0 = slice * k_chunk, k1 = k0 + k_chunk < k_len ? k0 + k_chunk : k_len;
    float acc[R][PER];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < PER; j++) acc[r][j] = 0.0f;
    if (valid) {
        const int sc_col = wc / (32 / PER);  // words never straddle a scale block
        const uint32_t *wp = words + wc;
        const float *sp = scales + sc_col;
        auto step = [&](uint32_t word, float scale, const float (&xk)[R]) {
            float q[PER];
#pragma unroll
            for (int j = 0; j < PER; j++)  // sign-extend field j: to the top of the word, then arithmetic shift back
                q[j] = (float)((int)(word << (32 - BITS * (j + 1))) >> (32 - BITS));
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float xs = __fmul_rn(xk[r], scale);
#pragma unroll
                for (int j = 0; j < PER; j++) acc[r][j] = __fadd_rn(acc[r][j], __fmul_rn(q[j], xs));
            }
        };
        int k = k0;
        for (; k + kPgUnroll <= k1; k += kPgUnroll) {
            uint32_t wv[kPgUnroll];
            float sv[kPgUnroll], xv[kPgUnroll][R];
#pragma unroll
            for (int u = 0; u < kPgUnroll; u++) {
                wv[u] = wp[(size_t)(k + u) * (size_t)n_words];
                sv[u] = sp[(size_t)(k + u) * (size_t)n_blocks];
#pragma unroll
                for (int r = 0; r < R; r++) xv[u][r] = xr[r][k + u];
            }
#pragma unroll
            for (int u = 0; u < kPgUnroll; u++) step(wv[u], sv[u], xv[u]);
        }
        for (; k < k1; k++) {
            float xk[R];
#pragma unroll
            for (int r = 0; r < R; r++) xk[r] = xr[r][k];
            step(wp[(size_t)k * (size_t)n_words], sp[(size_t)k * (size_t)n_blocks], xk);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < PER; j++) s_part[wave][r][lane][j] = acc[r][j];
    __syncthreads();
    if (wave == 0 && valid) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (row0 + r >= m) break;
            float *dst = out + (size_t)blockIdx.y * out_slice_stride + (size_t)(row0 + r) * (size_t)n_words * PER + (size_t)wc * PER;
#pragma unroll
            for (int j = 0; j < PER; j++) {
                float total = 0.0f;
#pragma unroll
                for (int w = 0; w < kPgWaves; w++) total = __fadd_rn(total, s_part[w][r][lane][j]);
                dst[j] = total;
            }
        }
    }
}

__global__ __launch_bounds__(256) void packed_gemv_sum_kernel(const float *__restrict__ partial, int slices, size_t n,
                                                              float *__restrict__ y) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    // ascending slices, eight loads out before the first add (a missing slice adds +0.0, which changes nothing)
    float total = 0.0f;
    for (int s0 = 0; s0 < slices; s0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = s0 + u < slices ? partial[(size_t)(s0 + u) * n + i] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) total = __fadd_rn(total, v[u]);
    }
    y[i] = total;
}

}  // namespace mummu

using namespace mummu;

struct mummu_packed_weight {
    uint32_t *words = nullptr;  // device [K][n_words]
    float *scales = nullptr;    // device [K][N/32]
    float *x = nullptr, *y = nullptr, *partial = nullptr;  // staging for the host-pointer call and the K partials
    int k = 0, n = 0, bits = 4, grid_k = 1, k_chunk = 0;
    bool owns_weight = true;  // false: words and scales are the caller's device buffers
    hipStream_t stream = nullptr;
    std::mutex mu;
    std::string error;
};

namespace {

constexpr int kMaxRows = 64;  // nn/packed_gemv.rs:138: row by row up to 64 rows
thread_local std::string g_packed_error;

int pfail(mummu_packed_weight *w, int code, const std::string &msg) {
    if (w) w->error = msg;
    g_packed_error = msg;
    return code;
}

int enqueue(mummu_packed_weight *w, const float *x_dev, int m, float *y_dev, hipStream_t s) {
    const int per = 32 / w->bits, n_words = w->n / per;
    const int rows_per = m == 1 ? 1 : (m == 2 ? 2 : 4);
    dim3 grid((unsigned)((n_words + 63) / 64), (unsigned)w->grid_k, (unsigned)((m + rows_per - 1) / rows_per)), block(64 * kPgWaves);
    const size_t out_n = (size_t)m * (size_t)w->n;
    float *dst = w->grid_k > 1 ? w->partial : y_dev;
#define MUMMU_PG(BITS, R)                                                                                                  \
    launch_kernel(packed_gemv_kernel<BITS, R>, grid, block, 0, s, (const uint32_t *)w->words, (const float *)w->scales, x_dev, m, \
                  w->k, n_words, w->n / 32, w->k_chunk, dst, out_n)
    if (w->bits == 4) {
        if (rows_per == 1) MUMMU_PG(4, 1);
        else if (rows_per == 2) MUMMU_PG(4, 2);
        else MUMMU_PG(4, 4);
    } else {
        if (rows_per == 1) MUMMU_PG(8, 1);
        else if (rows_per == 2) MUMMU_PG(8, 2);
        else MUMMU_PG(8, 4);
    }
#undef MUMMU_PG
    hipError_t e = hipGetLastError();
    if (e == hipSuccess && w->grid_k > 1) {
        launch_kernel(packed_gemv_sum_kernel, dim3((unsigned)((out_n + 255) / 256)), dim3(256), 0, s, (const float *)w->partial,
                      w->grid_k, out_n, y_dev);
        e = hipGetLastError();
    }
    if (e != hipSuccess) return pfail(w, MUMMU_ERR_DEVICE, std::string("packed gemv launch: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

}  // namespace

extern "C" {

const char *mummu_packed_last_error(void) { return g_packed_error.c_str(); }

static int packed_create(const uint32_t *words, const float *scales, int k, int n, int value_bits, bool on_device,
                         mummu_packed_weight **out) {
    if (!out) return pfail(nullptr, MUMMU_ERR_ARG, "null argument");
    *out = nullptr;
    if (!words || !scales) return pfail(nullptr, MUMMU_ERR_ARG, "null weight buffer");
    if (value_bits != 4 && value_bits != 8)
        return pfail(nullptr, MUMMU_ERR_TYPE, "packed weight: " + std::to_string(value_bits) + "-bit values are not supported (Q4S and Q8S are)");
    if (k < 1 || n < 1 || n % 32 != 0)
        return pfail(nullptr, MUMMU_ERR_SHAPE, "packed weight: [" + std::to_string(k) + ", " + std::to_string(n) +
                                                   "] needs K >= 1 and N a positive multiple of the 32-value scale block");
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices < 1) {
        (void)hipGetLastError();
        return pfail(nullptr, MUMMU_ERR_DEVICE, "no HIP device");
    }
    auto *w = new mummu_packed_weight();
    w->k = k;
    w->n = n;
    w->bits = value_bits;
    w->owns_weight = !on_device;
    const int per = 32 / value_bits, n_words = n / per;
    // K split over the grid: four workgroups per CU at one row (measured on Q4S [5120, 17408]: 21.3 us per call with
    // two, 19.4 with four; beyond that, and with slices shorter than 64 steps, only more partial sums to write and read
    // again), slices a whole number of unrolled steps and at least 64 steps long
    const int wg_x = (n_words + 63) / 64;
    int grid_k = (1024 + wg_x - 1) / wg_x;
    const int max_by_k = k / (64 * kPgWaves) > 0 ? k / (64 * kPgWaves) : 1;
    if (grid_k > max_by_k) grid_k = max_by_k;
    if (grid_k > 64) grid_k = 64;
    if (grid_k < 1) grid_k = 1;
    const int slices = grid_k * kPgWaves;
    w->k_chunk = ((k + slices - 1) / slices + kPgUnroll - 1) / kPgUnroll * kPgUnroll;
    w->grid_k = (k + w->k_chunk * kPgWaves - 1) / (w->k_chunk * kPgWaves);  // (rounding the slices up may empty the last workgroups)
    const size_t wb = sizeof(uint32_t) * (size_t)k * (size_t)n_words, sb = sizeof(float) * (size_t)k * (size_t)(n / 32);
    hipError_t e = hipSuccess;
    if (on_device) {
        w->words = const_cast<uint32_t *>(words);
        w->scales = const_cast<float *>(scales);
    } else {
        e = hipMalloc(&w->words, wb);
        if (e == hipSuccess) e = hipMalloc(&w->scales, sb);
    }
    if (e == hipSuccess) e = hipMalloc(&w->x, sizeof(float) * (size_t)kMaxRows * (size_t)k);
    if (e == hipSuccess) e = hipMalloc(&w->y, sizeof(float) * (size_t)kMaxRows * (size_t)n);
    if (e == hipSuccess) e = hipMalloc(&w->partial, sizeof(float) * (size_t)grid_k * (size_t)kMaxRows * (size_t)n);
    if (e == hipSuccess) e = hipStreamCreate(&w->stream);
    if (e == hipSuccess && !on_device) e = hipMemcpy(w->words, words, wb, hipMemcpyHostToDevice);
    if (e == hipSuccess && !on_device) e = hipMemcpy(w->scales, scales, sb, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        const std::string msg = std::string("packed weight: ") + hipGetErrorString(e);
        mummu_packed_weight_destroy(w);
        return pfail(nullptr, MUMMU_ERR_DEVICE, msg);
    }
    *out = w;
    return MUMMU_OK;
}

int mummu_packed_weight_create(const uint32_t *words, const float *scales, int k, int n, int value_bits,
                               mummu_packed_weight **out) {
    return packed_create(words, scales, k, n, value_bits, false, out);
}

int mummu_packed_weight_wrap_device(const uint32_t *words_dev, const float *scales_dev, int k, int n, int value_bits,
                                    mummu_packed_weight **out) {
    return packed_create(words_dev, scales_dev, k, n, value_bits, true, out);
}

void mummu_packed_weight_destroy(mummu_packed_weight *w) {
    if (!w) return;
    if (w->stream) {
        (void)hipStreamSynchronize(w->stream);
        (void)hipStreamDestroy(w->stream);
    }
    if (w->owns_weight) {
        (void)hipFree(w->words);
        (void)hipFree(w->scales);
    }
    (void)hipFree(w->x);
    (void)hipFree(w->y);
    (void)hipFree(w->partial);
    delete w;
}

uint64_t mummu_packed_weight_bytes(const mummu_packed_weight *w) {
    if (!w) return 0;
    return (uint64_t)w->k * (uint64_t)w->n * (uint64_t)w->bits / 8 + (uint64_t)w->k * (uint64_t)(w->n / 32) * 4;
}

int mummu_q4s_gemv(mummu_packed_weight *w, const float *x, int64_t m, int k, float *y) {
    if (!w) return pfail(nullptr, MUMMU_ERR_ARG, "null weight");
    std::lock_guard<std::mutex> lock(w->mu);
    if (k != w->k) return pfail(w, MUMMU_ERR_SHAPE, "input width " + std::to_string(k) + " does not match the weight's K " + std::to_string(w->k));
    if (m < 0 || m > kMaxRows) return pfail(w, MUMMU_ERR_TOKENS, std::to_string(m) + " rows: the packed GEMV takes 0 to 64 rows a call");
    if (m == 0) return MUMMU_OK;
    if (!x || !y) return pfail(w, MUMMU_ERR_ARG, "null buffer");
    hipError_t e = hipMemcpyAsync(w->x, x, sizeof(float) * (size_t)m * (size_t)k, hipMemcpyHostToDevice, w->stream);
    if (e != hipSuccess) return pfail(w, MUMMU_ERR_DEVICE, std::string("packed gemv upload: ") + hipGetErrorString(e));
    const int rc = enqueue(w, w->x, (int)m, w->y, w->stream);
    if (rc) return rc;
    e = hipMemcpyAsync(y, w->y, sizeof(float) * (size_t)m * (size_t)w->n, hipMemcpyDeviceToHost, w->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(w->stream);
    if (e != hipSuccess) return pfail(w, MUMMU_ERR_DEVICE, std::string("packed gemv: ") + hipGetErrorString(e));
    return MUMMU_OK;
}

int mummu_q4s_gemv_device(mummu_packed_weight *w, const float *x_dev, int64_t m, int k, float *y_dev, void *stream) {
    if (!w) return pfail(nullptr, MUMMU_ERR_ARG, "null weight");
    if (k != w->k) return pfail(w, MUMMU_ERR_SHAPE, "input width " + std::to_string(k) + " does not match the weight's K " + std::to_string(w->k));
    if (m < 0 || m > kMaxRows) return pfail(w, MUMMU_ERR_TOKENS, std::to_string(m) + " rows: the packed GEMV takes 0 to 64 rows a call");
    if (m == 0) return MUMMU_OK;
    if (!x_dev || !y_dev) return pfail(w, MUMMU_ERR_ARG, "null device pointer");
    return enqueue(w, x_dev, (int)m, y_dev, (hipStream_t)stream);
}

}  // extern "C"
