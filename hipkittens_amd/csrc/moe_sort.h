// Pieces of the stable counting sort of (token, choice) slots by expert that more than one kernel
// uses: the placement of one chunk of slots, and the whole sort of a small problem as one
// workgroup's work (the MoE layer runs it in the same launch as the quantization of its input).
#pragma once
#include "hk_device.h"

namespace hk {

constexpr int kSortChunk = 1024;   // slots per workgroup
constexpr int kSortMaxE = 512;

// Places the slots of chunk `chunk` (1024 consecutive slots, one workgroup of 4 waves):
// 16 rounds of 64 consecutive slots, wave w takes rounds 4w..4w+3. `first_pos(e)` = position of
// the chunk's first slot of expert e.
template <typename FirstPos>
__device__ __forceinline__ void sort_scatter_chunk(const int32_t* __restrict__ ids, int S, int E, int chunk,
                                                   int (&round_cnt)[16][kSortMaxE], FirstPos first_pos,
                                                   int32_t* __restrict__ sorted_slots,
                                                   int32_t* __restrict__ slot_to_pos) {
    const int lane = lane_id(), wv = threadIdx.x >> 6;
    const int base = chunk * kSortChunk;
    const int id_bits = E > 1 ? 32 - __clz(E - 1) : 0;
    for (int i = threadIdx.x; i < 16 * E; i += 256) round_cnt[i / E][i % E] = 0;   // later: exclusive prefix over rounds
    __syncthreads();
    int my_e[4], my_rank[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int rnd = wv * 4 + q;
        const int sidx = base + rnd * 64 + lane;
        int e = sidx < S ? ids[sidx] : -1;
        e = (unsigned)e < (unsigned)E ? e : -1;   // ids outside [0, E) take no part
        my_e[q] = e;
        // lanes of this round holding the same id, from one ballot per id bit; the stable rank
        // among equal ids is the number of such lanes below this one
        uint64_t same = __ballot(e >= 0);
        for (int b = 0; b < id_bits; ++b) {
            const bool bit = (e >> b) & 1;
            const uint64_t m = __ballot(bit);
            same &= bit ? m : ~m;
        }
        int rank = 0;
        if (e >= 0) {
            rank = __popcll(same & ((1ull << lane) - 1ull));
            if (rank == 0) round_cnt[rnd][e] = __popcll(same);
        }
        my_rank[q] = rank;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) {
        int run = first_pos(e);
#pragma unroll
        for (int rnd = 0; rnd < 16; ++rnd) {
            const int v = round_cnt[rnd][e];
            round_cnt[rnd][e] = run;
            run += v;
        }
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int rnd = wv * 4 + q;
        const int sidx = base + rnd * 64 + lane;
        if (my_e[q] >= 0) {
            const int pos = round_cnt[rnd][my_e[q]] + my_rank[q];
            sorted_slots[pos] = sidx;
            if (slot_to_pos) slot_to_pos[sidx] = pos;
        }
    }
}

// The whole sort in one launch for S <= 16384 slots (the layer of a few thousand tokens, where
// three launches and their gaps cost more than the work). No workgroup waits for another: each
// one histograms ALL ids itself (64 KiB from L2), split into slots before its chunk and the rest,
// scans the totals (workgroup 0 stores them as expert_offsets) and then places its own chunk as
// moe_sort_scatter_kernel does. Same result as the multi-launch path (stable, deterministic).
constexpr int kSortSmallMax = 16384;
struct MoeSortSmallLds {
    int round_cnt[16][kSortMaxE];
    int hist[2][kSortMaxE];   // [0]: slots before this chunk, [1]: the others; then first positions in [0]
    int wave_tot[4];
};
// Work of workgroup `chunk` (256 threads). `place` false: only the histogram and the scan (a chunk
// past the last slot then sees every slot as "before" it). On return thread t holds the ranges of
// experts 2t and 2t + 1 in the sorted order: [lo[j], hi[j]).
__device__ __forceinline__ void moe_sort_small_block(const int32_t* __restrict__ ids, int S, int E, int chunk,
                                                     bool place, int32_t* __restrict__ expert_offsets,
                                                     int32_t* __restrict__ sorted_slots,
                                                     int32_t* __restrict__ slot_to_pos, MoeSortSmallLds& lds,
                                                     int (&lo)[2], int (&hi)[2]) {
    auto& round_cnt = lds.round_cnt;
    auto& hist = lds.hist;
    auto& wave_tot = lds.wave_tot;
    const int lane = lane_id(), wv = threadIdx.x >> 6, tid = threadIdx.x;
    const int base = chunk * kSortChunk;
    // all ids of this thread are requested before the first one is used (16384 / 256 = 64 registers):
    // a loop of load - count - load would pay the memory latency once per trip
    int mine[kSortSmallMax / 256];
#pragma unroll
    for (int j = 0; j < kSortSmallMax / 256; ++j) {
        const int i = j * 256 + tid;
        mine[j] = i < S ? ids[i] : -1;
    }
    for (int e = tid; e < 2 * kSortMaxE; e += 256) (&hist[0][0])[e] = 0;
    __syncthreads();
    // a count does not depend on the order of the atomics
#pragma unroll
    for (int j = 0; j < kSortSmallMax / 256; ++j) {
        const int i = j * 256 + tid;
        if ((unsigned)mine[j] < (unsigned)E) atomicAdd(&hist[i < base ? 0 : 1][mine[j]], 1);
    }
    __syncthreads();
    // exclusive scan over e of the totals: thread t owns experts 2t, 2t + 1 (E <= 512)
    const int e0 = 2 * tid, e1 = 2 * tid + 1;
    const int t0 = e0 < E ? hist[0][e0] + hist[1][e0] : 0;
    const int t1 = e1 < E ? hist[0][e1] + hist[1][e1] : 0;
    int incl = t0 + t1;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int u = __shfl_up(incl, d, 64);
        if (lane >= d) incl += u;
    }
    if (lane == 63) wave_tot[wv] = incl;
    __syncthreads();
    int before = 0;
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2) before += w2 < wv ? wave_tot[w2] : 0;
    const int x0 = before + incl - t0 - t1, x1 = x0 + t0;
    if (e0 < E) hist[0][e0] += x0;
    if (e1 < E) hist[0][e1] += x1;
    lo[0] = x0; hi[0] = x1; lo[1] = x1; hi[1] = x1 + t1;
    if (chunk == 0 && place) {
        if (e0 < E) expert_offsets[e0] = x0;
        if (e1 < E) expert_offsets[e1] = x1;
        if (e0 == E - 1) expert_offsets[E] = x0 + t0;
        if (e1 == E - 1) expert_offsets[E] = x1 + t1;
    }
    __syncthreads();
    if (place)
        sort_scatter_chunk(ids, S, E, chunk, round_cnt, [&](int e) { return hist[0][e]; }, sorted_slots, slot_to_pos);
}


}  // namespace hk
