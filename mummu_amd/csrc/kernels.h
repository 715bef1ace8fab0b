// Host-callable launchers of the MoE kernels.  Each returns hipGetLastError() after the
// launch; shapes are validated by the caller (moe_api.cpp) before any launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mummu {

// error-flag words written by kernels (device int32[4])
enum : int { FLAG_NONFINITE = 0, FLAG_NONFINITE_INDEX = 1, FLAG_BAD_ID = 2 };

// dequant.hip -------------------------------------------------------------------------
// out[i] = dequantize(type, bytes)[i], bit-exact; nblocks blocks of the type.
hipError_t launch_dequantize(int type, const uint8_t *bytes, size_t nblocks, float *out, hipStream_t s);

// router.hip --------------------------------------------------------------------------
// logits[t, e] = <x[t, :], W[e, :]> in the fixed 512-partial order.  W row-major [E, H].
hipError_t launch_router_logits(const float *x, const void *w, int wtype, float *logits, int n, int hidden,
                                int n_experts, hipStream_t s);
// softmax -> top-k -> (re)normalise per token; one wave per token.
//   ids/weights [n, k] in slot order; hits (nullable) [E] += rows routed; flags see above.
hipError_t launch_route_topk(const float *logits, int n, int n_experts, int k, int flavour, int norm,
                             int32_t *ids, float *weights, unsigned long long *hits, int32_t *flags, hipStream_t s);
// x * rsqrt(mean(x^2) + eps) * gamma, one workgroup per token.
hipError_t launch_rmsnorm(const float *x, const float *gamma, float eps, int n, int hidden, float *out, hipStream_t s);
// dst = a + b (residual add), n elements.
hipError_t launch_add(const float *a, const float *b, float *dst, size_t n, hipStream_t s);

// experts.hip -------------------------------------------------------------------------
struct ExpertBanks {
    const uint8_t *gate, *up, *down;  // device, GGUF order
    int gate_type, up_type, down_type;
    int hidden, inter, n_experts;
};

// act[a, j] = silu(<gate_e[j,:], x_t>) * <up_e[j,:], x_t>  for assignment a = t*k + s,
// e = ids[a] (or fixed_expert >= 0 with token = a: the single-expert entry point).
hipError_t launch_gate_up(const ExpertBanks &b, const float *x, const int32_t *ids, int n_assign, int k,
                          int fixed_expert, float *act, int32_t *flags, hipStream_t s);
// y[a, c] = <down_e[c,:], act[a,:]>
hipError_t launch_down(const ExpertBanks &b, const float *act, const int32_t *ids, int n_assign, int fixed_expert,
                       float *y, hipStream_t s);
// out[t, c] = sum over the token's k slots in ASCENDING EXPERT ID of (w * y), two roundings.
// residual (nullable): out = residual + that sum.
hipError_t launch_combine(const float *y, const int32_t *ids, const float *weights, int n, int k, int hidden,
                          const float *residual, float *out, hipStream_t s);

}  // namespace mummu
