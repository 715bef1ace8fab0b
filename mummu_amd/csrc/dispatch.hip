// Token -> expert dispatch for batched (prefill) calls: a stable counting sort of the
// (token, slot) assignments by expert id, with the per-expert histograms, ranks and scans held
// in LDS.
//
// Reference: SparseMoePerExpert::route builds, per expert, the token rows it serves in
// token-major, slot-minor order (nn/moe.rs:275-285); RoutedExperts::apply_routing buckets
// (token, weight) the same way (models/qwen4exp/experts.rs:1108-1120).  The sort is stable, so
// every expert's segment lists its assignments in ascending a = token*k + slot, which is that
// order.
//
// Two small launches over chunks of 1024 assignments (one fused launch of one workgroup when there is a single
// chunk, where the launches themselves are most of the time):
//   count   per chunk: every assignment's rank among the chunk's assignments to the same expert
//           (wave ballots, then a prefix over the workgroup's 16 waves in LDS) and the chunk's
//           per-expert counts
//   scan + place   per chunk: per expert the count over the chunks before this one and the total, the
//           exclusive scan of the totals over experts (offsets), then
//           position = offsets[e] + rows of e in earlier chunks + rank.  Workgroup 0 also adds the totals to
//           the layer's hit counters when asked (8 atomics per token from the router would all land on the same
//           few cache lines) and writes the grouped GEMM's work list of (expert, first sorted position,
//           rows <= tile_rows) triples - every expert writes its own tiles at the position an exclusive scan of
//           the tile counts gives it
//
// Outputs (device):
//   offsets[E+1]      expert e owns sorted positions [offsets[e], offsets[e+1])
//   sorted[A]         sorted position -> assignment index a
//   inv[A]            assignment index a -> sorted position
//   tiles, n_tiles    the work list and its length
#include "device_utils.h"
#include "kernels.h"

namespace mummu {

constexpr int kDispatchThreads = 1024;
constexpr int kDispatchWaves = kDispatchThreads / 64;
constexpr int kDispatchMaxExperts = 512;

__global__ __launch_bounds__(kDispatchThreads) void dispatch_count_kernel(const int32_t *__restrict__ ids, int n_assign,
                                                                          int n_experts, int32_t *__restrict__ rank_out,
                                                                          int32_t *__restrict__ counts,
                                                                          int32_t *__restrict__ flags) {
    __shared__ int s_wave[kDispatchWaves][kDispatchMaxExperts];  // per-wave counts of this chunk
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk = blockIdx.x;
    for (int i = tid; i < kDispatchWaves * n_experts; i += kDispatchThreads) s_wave[i / n_experts][i % n_experts] = 0;
    __syncthreads();
    const int a = chunk * kDispatchThreads + tid;
    int e = a < n_assign ? ids[a] : -1;
    if (a < n_assign && (unsigned)e >= (unsigned)n_experts) {
        atomicAdd(&flags[FLAG_BAD_ID], 1);
        e = -1;
    }
    // rank among the lanes of this wave that hold the same expert, and that group's size
    int rank = 0;
    unsigned long long todo = __ballot(e >= 0);
    while (todo) {
        const int leader = (int)__builtin_ctzll(todo);
        const int le = __shfl(e, leader, 64);
        const unsigned long long same = __ballot(e == le);
        if (e == le) {
            rank = __builtin_popcountll(same & ((1ull << lane) - 1ull));
            if (rank == 0) s_wave[wave][e] = __builtin_popcountll(same);
        }
        todo &= ~same;
    }
    __syncthreads();
    if (e >= 0) {
        int before = 0;
        for (int w = 0; w < wave; w++) before += s_wave[w][e];
        rank_out[a] = before + rank;
    }
    for (int x = tid; x < n_experts; x += kDispatchThreads) {
        int total = 0;
#pragma unroll
        for (int w = 0; w < kDispatchWaves; w++) total += s_wave[w][x];
        counts[(size_t)chunk * n_experts + x] = total;
    }
}

// scan + place: every chunk's workgroup scans the (chunks x experts) counts for itself - a few thousand integers out
// of L2 - instead of waiting for a launch of one workgroup to do it once (a third launch costs 4-5 us, the repeated
// scan a fraction of that even at 64k tokens); workgroup 0 also writes offsets, the tile list and the hit counters.
__global__ __launch_bounds__(kDispatchThreads) void dispatch_scan_place_kernel(
    const int32_t *__restrict__ ids, int n_assign, int n_experts, int n_chunks, int tile_rows,
    const int32_t *__restrict__ rank_in, const int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
    int32_t *__restrict__ sorted, int32_t *__restrict__ inv, int32_t *__restrict__ tiles, int32_t *__restrict__ n_tiles,
    unsigned long long *__restrict__ hits) {
    __shared__ int s_carry[kDispatchMaxExperts / 64][2];
    __shared__ int s_pos[kDispatchMaxExperts];   // offsets[e] + rows of e in the chunks before this one
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk = blockIdx.x;
    const int e = tid;
    int total = 0, before = 0;
    if (e < n_experts) {
        for (int c = 0; c < n_chunks; c++) {
            const int v = counts[(size_t)c * n_experts + e];
            before += c < chunk ? v : 0;
            total += v;
        }
    }
    const int my_tiles = (total + tile_rows - 1) / tile_rows;
    int incl = total, incl_t = my_tiles;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64), up_t = __shfl_up(incl_t, off, 64);
        if (lane >= off) {
            incl += up;
            incl_t += up_t;
        }
    }
    if (lane == 63 && wave < kDispatchMaxExperts / 64) {
        s_carry[wave][0] = incl;
        s_carry[wave][1] = incl_t;
    }
    __syncthreads();
    if (e < n_experts) {
        int base = 0, base_t = 0;
        for (int w = 0; w < wave; w++) {
            base += s_carry[w][0];
            base_t += s_carry[w][1];
        }
        const int begin = base + incl - total;
        s_pos[e] = begin + before;
        if (chunk == 0) {
            if (hits) hits[e] += (unsigned long long)total;  // rows served per expert (nn/moe.rs:1562-1564)
            offsets[e] = begin;
            if (e == n_experts - 1) offsets[n_experts] = begin + total;
            if (tiles != nullptr) {
                int nt = base_t + incl_t - my_tiles;
                for (int r = 0; r < total; r += tile_rows, nt++) {
                    tiles[3 * nt] = e;
                    tiles[3 * nt + 1] = begin + r;
                    tiles[3 * nt + 2] = (total - r) < tile_rows ? (total - r) : tile_rows;
                }
                if (e == n_experts - 1) *n_tiles = base_t + incl_t;
            }
        }
    }
    __syncthreads();
    const int a = chunk * kDispatchThreads + tid;
    if (a >= n_assign) return;
    const int ea = ids[a];
    if ((unsigned)ea >= (unsigned)n_experts) return;
    const int pos = s_pos[ea] + rank_in[a];
    sorted[pos] = a;
    inv[a] = pos;
}

// The three steps above in one launch of one workgroup, for batches of at most kFusedChunks
// chunks: the per-chunk counts never leave LDS and every thread keeps its assignments' experts and
// ranks in registers between the steps.  Same outputs, element for element.  One workgroup takes
// about 7 us per chunk against 10 us for the two launches whatever the size, so this form only
// serves a single chunk (up to 1024 assignments).
constexpr int kFusedChunks = 1;

__global__ __launch_bounds__(kDispatchThreads) void dispatch_fused_kernel(
    const int32_t *__restrict__ ids, int n_assign, int n_experts, int tile_rows, int32_t *__restrict__ offsets,
    int32_t *__restrict__ sorted, int32_t *__restrict__ inv, int32_t *__restrict__ tiles, int32_t *__restrict__ n_tiles,
    unsigned long long *__restrict__ hits, int32_t *__restrict__ flags) {
    __shared__ int s_wave[kDispatchWaves][kDispatchMaxExperts];   // per-wave counts of the current chunk
    __shared__ int s_chunk[kFusedChunks][kDispatchMaxExperts];    // per-chunk counts, then exclusive running counts
    __shared__ int s_off[kDispatchMaxExperts];
    __shared__ int s_carry[kDispatchMaxExperts / 64][2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunks = (n_assign + kDispatchThreads - 1) / kDispatchThreads;
    int my_e[kFusedChunks], my_rank[kFusedChunks];
#pragma unroll
    for (int c = 0; c < kFusedChunks; c++) {
        my_e[c] = -1;
        my_rank[c] = 0;
        if (c >= chunks) continue;  // uniform over the workgroup
        for (int i = tid; i < kDispatchWaves * n_experts; i += kDispatchThreads) s_wave[i / n_experts][i % n_experts] = 0;
        __syncthreads();
        const int a = c * kDispatchThreads + tid;
        int e = a < n_assign ? ids[a] : -1;
        if (a < n_assign && (unsigned)e >= (unsigned)n_experts) {
            atomicAdd(&flags[FLAG_BAD_ID], 1);
            e = -1;
        }
        int rank = 0;
        unsigned long long todo = __ballot(e >= 0);
        while (todo) {
            const int leader = (int)__builtin_ctzll(todo);
            const int le = __shfl(e, leader, 64);
            const unsigned long long same = __ballot(e == le);
            if (e == le) {
                rank = __builtin_popcountll(same & ((1ull << lane) - 1ull));
                if (rank == 0) s_wave[wave][e] = __builtin_popcountll(same);
            }
            todo &= ~same;
        }
        __syncthreads();
        if (e >= 0) {
            int before = 0;
            for (int w = 0; w < wave; w++) before += s_wave[w][e];
            my_rank[c] = before + rank;
        }
        my_e[c] = e;
        for (int x = tid; x < n_experts; x += kDispatchThreads) {
            int total = 0;
#pragma unroll
            for (int w = 0; w < kDispatchWaves; w++) total += s_wave[w][x];
            s_chunk[c][x] = total;
        }
        __syncthreads();  // s_wave is cleared again for the next chunk
    }
    // running counts over chunks, offsets over experts, the work list (threads = experts)
    const int e = tid;
    int total = 0;
    if (e < n_experts) {
        for (int c = 0; c < chunks; c++) {
            const int v = s_chunk[c][e];
            s_chunk[c][e] = total;
            total += v;
        }
    }
    const int my_tiles = (total + tile_rows - 1) / tile_rows;
    int incl = total, incl_t = my_tiles;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64), up_t = __shfl_up(incl_t, off, 64);
        if (lane >= off) {
            incl += up;
            incl_t += up_t;
        }
    }
    if (lane == 63 && wave < kDispatchMaxExperts / 64) {
        s_carry[wave][0] = incl;
        s_carry[wave][1] = incl_t;
    }
    __syncthreads();
    if (e < n_experts) {
        int base = 0, base_t = 0;
        for (int w = 0; w < wave; w++) {
            base += s_carry[w][0];
            base_t += s_carry[w][1];
        }
        const int begin = base + incl - total;
        if (hits) hits[e] += (unsigned long long)total;
        offsets[e] = begin;
        s_off[e] = begin;
        if (e == n_experts - 1) offsets[n_experts] = begin + total;
        if (tiles != nullptr) {
            int nt = base_t + incl_t - my_tiles;
            for (int r = 0; r < total; r += tile_rows, nt++) {
                tiles[3 * nt] = e;
                tiles[3 * nt + 1] = begin + r;
                tiles[3 * nt + 2] = (total - r) < tile_rows ? (total - r) : tile_rows;
            }
            if (e == n_experts - 1) *n_tiles = base_t + incl_t;
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < kFusedChunks; c++) {
        if (c >= chunks || my_e[c] < 0) continue;
        const int a = c * kDispatchThreads + tid;
        const int pos = s_off[my_e[c]] + s_chunk[c][my_e[c]] + my_rank[c];
        sorted[pos] = a;
        inv[a] = pos;
    }
}

// The work list of ONE expert that serves every row in order (the shared expert of a Qwen-style
// block on the batched path): sorted[i] = i, tiles of tile_rows rows of expert 0.
__global__ __launch_bounds__(256) void identity_tiles_kernel(int n, int tile_rows, int32_t *__restrict__ sorted,
                                                             int32_t *__restrict__ tiles, int32_t *__restrict__ n_tiles) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) sorted[i] = i;
    const int nt = (n + tile_rows - 1) / tile_rows;
    if (i < nt) {
        tiles[3 * i] = 0;
        tiles[3 * i + 1] = i * tile_rows;
        tiles[3 * i + 2] = (n - i * tile_rows) < tile_rows ? (n - i * tile_rows) : tile_rows;
    }
    if (i == 0) *n_tiles = nt;
}

hipError_t launch_identity_tiles(int n, int tile_rows, int32_t *sorted, int32_t *tiles, int32_t *n_tiles, hipStream_t s) {
    if (n <= 0 || tile_rows < 1) return hipErrorInvalidValue;
    launch_kernel(identity_tiles_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, tile_rows, sorted, tiles, n_tiles);
    return hipGetLastError();
}

size_t dispatch_scratch_ints(int n_assign, int n_experts) {
    const size_t chunks = ((size_t)n_assign + kDispatchThreads - 1) / kDispatchThreads;
    return (size_t)n_assign + chunks * (size_t)n_experts;
}

hipError_t launch_dispatch(const int32_t *ids, int n_assign, int n_experts, int tile_rows, int32_t *offsets,
                           int32_t *sorted, int32_t *inv, int32_t *tiles, int32_t *n_tiles, int32_t *scratch,
                           unsigned long long *hits, int32_t *flags, hipStream_t s) {
    if (n_assign <= 0) return hipSuccess;
    if (n_experts > kDispatchMaxExperts || tile_rows < 1) return hipErrorInvalidValue;
    const int chunks = (n_assign + kDispatchThreads - 1) / kDispatchThreads;
    if (chunks <= kFusedChunks) {
        launch_kernel(dispatch_fused_kernel, dim3(1), dim3(kDispatchThreads), 0, s, ids, n_assign, n_experts, tile_rows, offsets,
                      sorted, inv, tiles, n_tiles, hits, flags);
        return hipGetLastError();
    }
    int32_t *rank = scratch, *counts = scratch + n_assign;
    // per-kernel timing brackets the two launches as one: start from the first, stop from the last
    const LaunchTiming timing = g_launch_timing;
    g_launch_timing.stop = nullptr;
    launch_kernel(dispatch_count_kernel, dim3(chunks), dim3(kDispatchThreads), 0, s, ids, n_assign, n_experts, rank, counts,
                  flags);
    g_launch_timing.start = nullptr;
    g_launch_timing.stop = timing.stop;
    launch_kernel(dispatch_scan_place_kernel, dim3(chunks), dim3(kDispatchThreads), 0, s, ids, n_assign, n_experts, chunks,
                  tile_rows, (const int32_t *)rank, (const int32_t *)counts, offsets, sorted, inv, tiles, n_tiles, hits);
    g_launch_timing = timing;
    return hipGetLastError();
}

}  // namespace mummu
