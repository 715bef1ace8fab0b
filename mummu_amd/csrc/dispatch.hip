// Token -> expert dispatch for batched (prefill) calls: a stable counting sort of the
// (token, slot) assignments by expert id, with the per-expert histogram, its exclusive scan
// and the running cursors all held in LDS.
//
// Reference: SparseMoePerExpert::route builds, per expert, the token rows it serves in
// token-major, slot-minor order (nn/moe.rs:275-285); RoutedExperts::apply_routing buckets
// (token, weight) the same way (models/qwen4exp/experts.rs:1108-1120).  The sort is stable, so
// every expert's segment lists its assignments in ascending a = token*k + slot, which is that
// order.
//
// Outputs (device):
//   offsets[E+1]      exclusive scan of the histogram: expert e owns sorted positions
//                     [offsets[e], offsets[e+1])
//   sorted[A]         sorted position -> assignment index a
//   inv[A]            assignment index a -> sorted position
//   tiles             the work list of the grouped GEMM: for every expert with rows, its
//                     segments of at most `tile_rows` sorted positions, as
//                     (expert, first position, rows) triples; tiles[0..3*n) then n in *n_tiles
#include "device_utils.h"
#include "kernels.h"

namespace mummu {

constexpr int kDispatchThreads = 1024;
constexpr int kDispatchWaves = kDispatchThreads / 64;
constexpr int kDispatchMaxExperts = 512;

__global__ __launch_bounds__(kDispatchThreads) void dispatch_kernel(const int32_t *__restrict__ ids, int n_assign,
                                                                    int n_experts, int tile_rows,
                                                                    int32_t *__restrict__ offsets,
                                                                    int32_t *__restrict__ sorted,
                                                                    int32_t *__restrict__ inv,
                                                                    int32_t *__restrict__ tiles,
                                                                    int32_t *__restrict__ n_tiles,
                                                                    int32_t *__restrict__ flags) {
    __shared__ int s_hist[kDispatchMaxExperts];                   // per-expert counts, then exclusive offsets
    __shared__ int s_cursor[kDispatchMaxExperts];                 // next free position of each expert
    __shared__ int s_wave[kDispatchWaves][kDispatchMaxExperts];   // per-wave counts of the current round
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    for (int e = tid; e < n_experts; e += kDispatchThreads) s_hist[e] = 0;
    __syncthreads();
    for (int a = tid; a < n_assign; a += kDispatchThreads) {
        const int e = ids[a];
        if ((unsigned)e < (unsigned)n_experts) atomicAdd(&s_hist[e], 1);
        else atomicAdd(&flags[FLAG_BAD_ID], 1);
    }
    __syncthreads();
    // exclusive scan over experts (a few hundred entries: one wave, sequential per 64-chunk)
    if (wave == 0) {
        int carry = 0;
        for (int base = 0; base < n_experts; base += 64) {
            const int e = base + lane;
            const int c = e < n_experts ? s_hist[e] : 0;
            int incl = c;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int up = __shfl_up(incl, off, 64);
                if (lane >= off) incl += up;
            }
            if (e < n_experts) {
                s_hist[e] = carry + incl - c;
                s_cursor[e] = carry + incl - c;
                offsets[e] = carry + incl - c;
            }
            carry += __shfl(incl, 63, 64);
        }
        if (lane == 0) offsets[n_experts] = carry;
    }
    __syncthreads();

    // stable placement, kDispatchThreads assignments per round in ascending a
    for (int base = 0; base < n_assign; base += kDispatchThreads) {
        for (int i = tid; i < kDispatchWaves * kDispatchMaxExperts; i += kDispatchThreads) (&s_wave[0][0])[i] = 0;
        __syncthreads();
        const int a = base + tid;
        int e = a < n_assign ? ids[a] : -1;
        if ((unsigned)e >= (unsigned)n_experts) e = -1;
        // rank among the lanes of this wave that hold the same expert, and that group's size
        int rank = 0, cnt = 0;
        unsigned long long todo = __ballot(e >= 0);
        while (todo) {
            const int leader = (int)__builtin_ctzll(todo);
            const int le = __shfl(e, leader, 64);
            const unsigned long long same = __ballot(e == le);
            if (e == le) {
                rank = __builtin_popcountll(same & ((1ull << lane) - 1ull));
                cnt = __builtin_popcountll(same);
                if (rank == 0) s_wave[wave][e] = cnt;
            }
            todo &= ~same;
        }
        __syncthreads();
        if (e >= 0) {
            int before = 0;
            for (int w = 0; w < wave; w++) before += s_wave[w][e];
            const int pos = s_cursor[e] + before + rank;
            sorted[pos] = a;
            inv[a] = pos;
        }
        __syncthreads();
        for (int x = tid; x < n_experts; x += kDispatchThreads) {
            int total = 0;
            for (int w = 0; w < kDispatchWaves; w++) total += s_wave[w][x];
            s_cursor[x] += total;
        }
        __syncthreads();
    }

    // work list of the grouped GEMM
    if (tid == 0 && tiles != nullptr) {
        int nt = 0;
        for (int e = 0; e < n_experts; e++) {
            const int begin = s_hist[e], stop = s_cursor[e];  // after placement a cursor is its segment's end
            for (int r = begin; r < stop; r += tile_rows) {
                tiles[3 * nt] = e;
                tiles[3 * nt + 1] = r;
                tiles[3 * nt + 2] = (stop - r) < tile_rows ? (stop - r) : tile_rows;
                nt++;
            }
        }
        *n_tiles = nt;
    }
}

hipError_t launch_dispatch(const int32_t *ids, int n_assign, int n_experts, int tile_rows, int32_t *offsets,
                           int32_t *sorted, int32_t *inv, int32_t *tiles, int32_t *n_tiles, int32_t *flags,
                           hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    if (n_experts > kDispatchMaxExperts || tile_rows < 1) return hipErrorInvalidValue;
    launch_kernel(dispatch_kernel, dim3(1), dim3(kDispatchThreads), 0, s, ids, n_assign, n_experts, tile_rows, offsets, sorted, inv,
                                                               tiles, n_tiles, flags);
    return hipGetLastError();
}

}  // namespace mummu
