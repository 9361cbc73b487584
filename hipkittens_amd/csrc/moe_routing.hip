// MoE routing for gfx950: top-k selection (softmax and group-limited sigmoid) and the stable
// counting sort of (token, choice) slots by expert. All bandwidth / latency bound; one wave per
// token, wavefront shuffles and ballots, coalesced HBM access.
//
// The reference has no MoE code (no counterpart to cite). Integer outputs are specified to be
// bit-exact against the CPU oracle: ties go to the lower expert id, the sort is stable, and the
// sigmoid used for selection is a fixed sequence of correctly rounded fp32 operations.
#include "hk_device.h"
#include "moe_sort.h"
#include "../../include/hk355.h"

// This file must be compiled with -ffp-contract=off (hipkittens_amd/build.py does): the routing
// arithmetic is specified as separately rounded fp32 operations, and HIP's __fmul_rn / __fadd_rn
// are plain operators that the compiler would otherwise fuse into FMAs.

namespace hk {

// ---------------------------------------------------------------------------------- helpers
// Monotonic key: larger float -> larger key; -0.0 and +0.0 compare equal.
__device__ __forceinline__ uint32_t float_key(float x) {
    uint32_t u = __float_as_uint(x);
    if (x == 0.0f) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// (key, expert id) packed so that max() picks the larger key and, on ties, the lower id.
__device__ __forceinline__ uint64_t pack_choice(float x, int id) {
    return ((uint64_t)float_key(x) << 32) | (uint32_t)(0x7fffffff - id);
}
__device__ __forceinline__ int choice_id(uint64_t c) { return 0x7fffffff - (int)(uint32_t)c; }

__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint64_t o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}
__device__ __forceinline__ float wave_sum_f32_ordered(float v, int k, int lane) {
    // sum of lanes 0..k-1 in lane order (k <= 64), the same order the oracle uses
    float tot = 0.f;
    for (int j = 0; j < k; ++j) tot = __fadd_rn(tot, __shfl(v, j, 64));
    return tot;
}

// exp(x) for x in [-87, 0] and the sigmoid built on it: fixed fp32 operation sequence, no
// contraction, so that CPU and GPU agree bit for bit.
__device__ __forceinline__ float exp_neg_f32(float x) {
    x = fmaxf(x, -87.0f);
    const float n = rintf(__fmul_rn(x, 1.4426950408889634f));
    float r = __fsub_rn(x, __fmul_rn(n, 0.693145751953125f));
    r = __fsub_rn(r, __fmul_rn(n, 1.4286068203094172e-06f));
    float p = 1.0f / 720;
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 120);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 24);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 6);
    p = __fadd_rn(__fmul_rn(p, r), 0.5f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f);
    return ldexpf(p, (int)n);
}
__device__ __forceinline__ float sigmoid_f32(float x) {
    const float e = exp_neg_f32(-fabsf(x));
    const float d = __fadd_rn(1.0f, e);
    return __fdiv_rn(x >= 0.f ? 1.0f : e, d);   // 1 / d or e / d: one division
}

constexpr int kMaxPerLane = 8;  // experts per lane: E <= 512

// ------------------------------------------------------------------------- top-k softmax
// LPT lanes per token (64 / LPT tokens per wave): LPT = 16 when E <= 128 and k <= 16, so that a
// wave's loads cover four token rows, else one wave per token. ids[t, j] = j-th largest logit
// (ties -> lower id); w = softmax over the k selected logits.
template <int LPT>
__global__ __launch_bounds__(256) void moe_topk_softmax_kernel(const float* __restrict__ logits, int T,
                                                               int E, int k, int32_t* __restrict__ ids,
                                                               float* __restrict__ w) {
    constexpr int TPW = 64 / LPT;  // tokens per wave
    const int lane = lane_id(), sub = lane % LPT;
    const int t = (blockIdx.x * 4 + (threadIdx.x >> 6)) * TPW + lane / LPT;
    const bool live = t < T;
    const float* row = logits + (size_t)(live ? t : 0) * E;
    // Selection in 32-bit operations: per round the largest key over the token's lanes, then the
    // lowest id among its holders (the order of pack_choice). Key 0 = taken or absent (the key of a
    // number is never 0).
    uint32_t ck[kMaxPerLane];
    const int per = (E + LPT - 1) / LPT;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = i * LPT + sub;  // coalesced within the token's row
        ck[i] = (live && i < per && e < E) ? float_key(row[e]) : 0u;
    }
    float my_logit = 0.f, top_logit = 0.f;
    int my_id = 0;
    for (int j = 0; j < k; ++j) {
        uint32_t bk = 0;
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i) bk = ck[i] > bk ? ck[i] : bk;
#pragma unroll
        for (int off = LPT / 2; off >= 1; off >>= 1) {
            const uint32_t o = __shfl_xor(bk, off, 64);
            bk = o > bk ? o : bk;
        }
        int id = 0x7fffffff;
#pragma unroll
        for (int i = kMaxPerLane - 1; i >= 0; --i) id = ck[i] == bk ? i * LPT + sub : id;
#pragma unroll
        for (int off = LPT / 2; off >= 1; off >>= 1) {
            const int o = __shfl_xor(id, off, 64);
            id = o < id ? o : id;
        }
        if (!live) id = 0;
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i)
            if (i * LPT + sub == id) ck[i] = 0u;
        // the logit back from its key (exact; -0 comes back as +0, which the softmax cannot tell apart):
        // no dependent reload of row[id]
        const float v = __uint_as_float((bk & 0x80000000u) ? bk ^ 0x80000000u : ~bk);
        if (j == 0) top_logit = v;
        if (sub == j) { my_logit = v; my_id = id; }
    }
    const float ex = sub < k ? expf(my_logit - top_logit) : 0.f;
    float tot = ex;
#pragma unroll
    for (int off = LPT / 2; off >= 1; off >>= 1) tot += __shfl_xor(tot, off, 64);
    if (live && sub < k) {
        ids[(size_t)t * k + sub] = my_id;
        w[(size_t)t * k + sub] = ex / tot;
    }
}

// ------------------------------------------------------------- group-limited sigmoid top-k
__global__ __launch_bounds__(256) void moe_topk_grouped_sigmoid_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int T, int E, int k, int n_group,
    int topk_group, float routed_scale, int32_t* __restrict__ ids, float* __restrict__ w) {
    const int lane = lane_id();
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* row = logits + (size_t)t * E;
    const int gs = E / n_group;
    const int per = (E + 63) / 64;
    float s[kMaxPerLane], c[kMaxPerLane];
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = i * 64 + lane;
        s[i] = 0.f; c[i] = 0.f;
        if (i < per && e < E) {
            s[i] = sigmoid_f32(row[e]);
            c[i] = bias ? __fadd_rn(s[i], bias[e]) : s[i];
        }
    }
    // group scores: sum of the two largest c in each group. Lane g (< n_group) ends up owning
    // group g's score.
    float gscore = -INFINITY;
    for (int grp = 0; grp < n_group; ++grp) {
        uint64_t best1 = 0, best2 = 0;
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i) {
            const int e = i * 64 + lane;
            if (i < per && e < E && e / gs == grp) {
                const uint64_t p = pack_choice(c[i], e);
                if (p > best1) { best2 = best1; best1 = p; } else if (p > best2) best2 = p;
            }
        }
        const uint64_t m1 = wave_max_u64(best1);
        const uint64_t mine = (best1 == m1) ? best2 : best1;  // runner-up candidates
        const uint64_t m2 = wave_max_u64(mine);
        // recover the two values from their owners
        float v1 = 0.f, v2 = 0.f;
        const int id1 = choice_id(m1), id2 = choice_id(m2);
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i) {
            const int e = i * 64 + lane;
            if (i < per && e == id1) v1 = c[i];
            if (i < per && e == id2) v2 = c[i];
        }
        v1 = __shfl(v1, id1 & 63, 64);
        v2 = __shfl(v2, id2 & 63, 64);
        const float sc = gs >= 2 ? __fadd_rn(v1, v2) : v1;
        if (lane == grp) gscore = sc;
    }
    // keep the topk_group best groups (ties -> lower group id)
    uint64_t gc = lane < n_group ? pack_choice(gscore, lane) : 0ull;
    uint64_t keep_mask = 0;
    for (int j = 0; j < topk_group; ++j) {
        const uint64_t b = wave_max_u64(gc);
        if (gc == b) gc = 0ull;
        keep_mask |= 1ull << choice_id(b);
    }
    // top-k of c among the kept groups
    uint64_t cand[kMaxPerLane];
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = i * 64 + lane;
        const bool ok = i < per && e < E && ((keep_mask >> (e / gs)) & 1ull);
        cand[i] = ok ? pack_choice(c[i], e) : 0ull;
    }
    float my_s = 0.f;
    int my_id = 0;
    for (int j = 0; j < k; ++j) {
        uint64_t best = 0;
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i) best = cand[i] > best ? cand[i] : best;
        best = wave_max_u64(best);
        const int id = choice_id(best);
        float sv = 0.f;
#pragma unroll
        for (int i = 0; i < kMaxPerLane; ++i)
            if (cand[i] == best) { cand[i] = 0ull; sv = s[i]; }
        sv = __shfl(sv, id & 63, 64);
        if (lane == j) { my_s = sv; my_id = id; }
    }
    const float tot = wave_sum_f32_ordered(my_s, k, lane);
    if (lane < k) {
        ids[(size_t)t * k + lane] = my_id;
        w[(size_t)t * k + lane] = __fmul_rn(__fdiv_rn(my_s, tot), routed_scale);
    }
}

// The same routing with 16 lanes per token (4 tokens per wave), for E = 16 * PER (PER <= 16) experts
// whose groups are runs of whole lanes: lane `sub` of a token holds the experts [sub * PER, +PER),
// a group is LG = (E / n_group) / PER adjacent lanes (a power of two). Reductions then run over
// 16 lanes and serve four tokens at once; the two best of a group are merged from per-lane pairs.
// Same operation sequence per value as the kernel above, so the results are bit-identical to it.
template <int PER>
__global__ __launch_bounds__(256) void moe_topk_grouped_sigmoid16_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int T, int k, int lg_shift,
    int topk_group, float routed_scale, int32_t* __restrict__ ids, float* __restrict__ w) {
    constexpr int E = 16 * PER;
    const int lane = lane_id(), sub = lane & 15, seg = lane & ~15;
    const int t = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);
    const bool live = t < T;
    const float* row = logits + (size_t)(live ? t : 0) * E + sub * PER;
    const int grp = sub >> lg_shift;   // this lane's group
    float s[PER];
    uint64_t cand[PER];
    uint64_t best1 = 0, best2 = 0;     // the lane's two best (c, id) choices
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = sub * PER + i;
        s[i] = sigmoid_f32(row[i]);
        const float c = bias ? __fadd_rn(s[i], bias[e]) : s[i];
        cand[i] = pack_choice(c, e);
        if (cand[i] > best1) { best2 = best1; best1 = cand[i]; } else if (cand[i] > best2) best2 = cand[i];
    }
    // merge the pairs over the LG lanes of the group: afterwards every lane of a group holds the
    // group's two best
    for (int off = 1; off < (1 << lg_shift); off <<= 1) {
        const uint64_t o1 = __shfl_xor(best1, off, 64), o2 = __shfl_xor(best2, off, 64);
        const uint64_t hi = best1 > o1 ? best1 : o1, lo = best1 > o1 ? o1 : best1;
        const uint64_t second = best2 > o2 ? best2 : o2;
        best1 = hi;
        best2 = lo > second ? lo : second;
    }
    auto key_value = [](uint64_t ch) {
        const uint32_t key = (uint32_t)(ch >> 32);
        return __uint_as_float((key & 0x80000000u) ? key ^ 0x80000000u : ~key);
    };
    const float gscore = PER << lg_shift >= 2 ? __fadd_rn(key_value(best1), key_value(best2)) : key_value(best1);
    // keep the topk_group best groups (ties -> lower group id); the lanes of a group carry the same choice
    uint64_t gc = pack_choice(gscore, grp);
    bool kept = false;
    for (int j = 0; j < topk_group; ++j) {
        uint64_t b = gc;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) {
            const uint64_t o = __shfl_xor(b, off, 64);
            b = o > b ? o : b;
        }
        if (gc == b) { gc = 0ull; kept = true; }
    }
    // The k best of the kept groups, in the order of the (key, id) pairs: per round the largest 32-bit
    // key over the token's 16 lanes, then the lowest id among its holders (ids grow with i and with
    // the lane), all in 32-bit operations. A key of 0 marks a choice that is taken or not kept (the
    // key of a real score is never 0).
    uint32_t ck[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) ck[i] = kept ? (uint32_t)(cand[i] >> 32) : 0u;
    float my_s = 0.f;
    int my_id = 0;
    for (int j = 0; j < k; ++j) {
        uint32_t bk = 0;
#pragma unroll
        for (int i = 0; i < PER; ++i) bk = ck[i] > bk ? ck[i] : bk;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) {
            const uint32_t o = __shfl_xor(bk, off, 64);
            bk = o > bk ? o : bk;
        }
        int id = 0x7fffffff;
#pragma unroll
        for (int i = PER - 1; i >= 0; --i) id = ck[i] == bk ? sub * PER + i : id;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) {
            const int o = __shfl_xor(id, off, 64);
            id = o < id ? o : id;
        }
        float sv = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (sub * PER + i == id) { ck[i] = 0u; sv = s[i]; }
        sv = __shfl(sv, seg + id / PER, 64);
        if (sub == j) { my_s = sv; my_id = id; }
    }
    // sum of the k selected scores in selection order
    float tot = 0.f;
    for (int j = 0; j < k; ++j) tot = __fadd_rn(tot, __shfl(my_s, seg + j, 64));
    if (live && sub < k) {
        ids[(size_t)t * k + sub] = my_id;
        w[(size_t)t * k + sub] = __fmul_rn(__fdiv_rn(my_s, tot), routed_scale);
    }
}

// --------------------------------------------------------------------------------- sort
// Stable counting sort of S = T*k slots by expert id, four launches:
//   count   : per-chunk histogram (chunk = 1024 consecutive slots) -> ws[chunk][E]
//   scan    : ws[chunk][e] := slots of expert e in earlier chunks (one workgroup per expert);
//   offsets : expert_offsets[0..E] from the per-expert totals
//   scatter : position of a slot = expert_offsets[e] + ws[chunk][e] + earlier slots of e in the chunk
// The within-chunk rank comes from wave ballots in slot order, never from atomics' arrival
// order, so the result is deterministic and stable.

__global__ __launch_bounds__(256) void moe_sort_count_kernel(const int32_t* __restrict__ ids, int S,
                                                             int E, int32_t* __restrict__ ws) {
    __shared__ int cnt[kSortMaxE];
    for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
    __syncthreads();
    const int base = blockIdx.x * kSortChunk;
#pragma unroll
    for (int i = 0; i < kSortChunk / 256; ++i) {
        const int sidx = base + i * 256 + threadIdx.x;
        if (sidx < S) {
            const int e = ids[sidx];
            if ((unsigned)e < (unsigned)E) atomicAdd(&cnt[e], 1);   // ids outside [0, E) take no part
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) ws[(size_t)blockIdx.x * E + e] = cnt[e];
}

// One workgroup per expert: exclusive prefix of that expert's per-chunk counts over the chunks
// (ws[chunk][e] := number of slots of e in earlier chunks) and the expert's total.
__global__ __launch_bounds__(256) void moe_sort_scan_kernel(int32_t* __restrict__ ws, int nchunks, int E,
                                                            int32_t* __restrict__ totals) {
    __shared__ int part[256];
    const int e = blockIdx.x, t = threadIdx.x;
    int carry = 0;
    for (int c0 = 0; c0 < nchunks; c0 += 256) {
        const int c = c0 + t;
        const int v = c < nchunks ? ws[(size_t)c * E + e] : 0;
        part[t] = v;
        __syncthreads();
        for (int d = 1; d < 256; d <<= 1) {
            const int u = t >= d ? part[t - d] : 0;
            __syncthreads();
            part[t] += u;
            __syncthreads();
        }
        if (c < nchunks) ws[(size_t)c * E + e] = carry + part[t] - v;
        carry += part[255];
        __syncthreads();
    }
    if (t == 0) totals[e] = carry;
}

// The scan above and the exclusive prefix sum of the totals (expert_offsets[0..E]) in one workgroup
// when there are few chunks: thread e walks expert e's per-chunk counts, then the workgroup scans the totals.
constexpr int kSortFusedChunks = 64;
__global__ __launch_bounds__(512) void moe_sort_scan_offsets_kernel(int32_t* __restrict__ ws, int nchunks, int E,
                                                                    int32_t* __restrict__ expert_offsets) {
    __shared__ int scan[512];
    const int e = threadIdx.x;
    int total = 0;
    if (e < E) {
        // all 64 loads in flight at once through a descriptor of the counts' size: chunks beyond nchunks read as
        // zero and their stores are dropped by the range check, so no load or store carries a condition of its own
        // (64 wave-uniform conditions kept live cost 40 spilled scalar registers)
        const __amdgpu_buffer_rsrc_t counts =
            __builtin_amdgcn_make_buffer_rsrc(ws, 0, nchunks * E * (int)sizeof(int32_t), 0x00020000);
        const int pitch = E * (int)sizeof(int32_t);
        int v[kSortFusedChunks];
#pragma unroll
        for (int c = 0; c < kSortFusedChunks; ++c)
            v[c] = __builtin_amdgcn_raw_buffer_load_b32(counts, c * pitch + e * (int)sizeof(int32_t), 0, 0);
#pragma unroll
        for (int c = 0; c < kSortFusedChunks; ++c) {
            __builtin_amdgcn_raw_buffer_store_b32(total, counts, c * pitch + e * (int)sizeof(int32_t), 0, 0);
            total += v[c];
        }
    }
    scan[e] = total;
    __syncthreads();
    for (int d = 1; d < 512; d <<= 1) {
        const int u = e >= d ? scan[e - d] : 0;
        __syncthreads();
        scan[e] += u;
        __syncthreads();
    }
    if (e < E) expert_offsets[e] = scan[e] - total;
    if (e == 511) expert_offsets[E] = scan[511];
}

__global__ __launch_bounds__(256) void moe_sort_scatter_kernel(const int32_t* __restrict__ ids, int S, int E,
                                                               const int32_t* __restrict__ ws,
                                                               const int32_t* __restrict__ expert_offsets,
                                                               int32_t* __restrict__ sorted_slots,
                                                               int32_t* __restrict__ slot_to_pos) {
    __shared__ int round_cnt[16][kSortMaxE];
    const int chunk = blockIdx.x;
    sort_scatter_chunk(ids, S, E, chunk, round_cnt,
                       [&](int e) { return expert_offsets[e] + ws[(size_t)chunk * E + e]; }, sorted_slots,
                       slot_to_pos);
}

// moe_sort_scatter_kernel for many chunks: expert_offsets does not exist yet; every workgroup scans
// the per-expert totals itself (E <= 512 values, two per thread) and workgroup 0 stores the result,
// which saves a launch for the prefix sum of the totals.
__global__ __launch_bounds__(256) void moe_sort_scatter_totals_kernel(const int32_t* __restrict__ ids, int S, int E,
                                                                      const int32_t* __restrict__ ws,
                                                                      const int32_t* __restrict__ totals,
                                                                      int32_t* __restrict__ expert_offsets,
                                                                      int32_t* __restrict__ sorted_slots,
                                                                      int32_t* __restrict__ slot_to_pos) {
    __shared__ int round_cnt[16][kSortMaxE];
    __shared__ int first[kSortMaxE];
    __shared__ int wave_tot[4];
    const int lane = lane_id(), wv = threadIdx.x >> 6, tid = threadIdx.x;
    const int chunk = blockIdx.x;
    const int e0 = 2 * tid, e1 = 2 * tid + 1;
    const int t0 = e0 < E ? totals[e0] : 0, t1 = e1 < E ? totals[e1] : 0;
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
    if (e0 < E) first[e0] = x0 + ws[(size_t)chunk * E + e0];
    if (e1 < E) first[e1] = x1 + ws[(size_t)chunk * E + e1];
    if (chunk == 0) {
        if (e0 < E) expert_offsets[e0] = x0;
        if (e1 < E) expert_offsets[e1] = x1;
        if (e0 == E - 1) expert_offsets[E] = x0 + t0;
        if (e1 == E - 1) expert_offsets[E] = x1 + t1;
    }
    __syncthreads();
    sort_scatter_chunk(ids, S, E, chunk, round_cnt, [&](int e) { return first[e]; }, sorted_slots, slot_to_pos);
}

// The whole sort in one launch for S <= kSortSmallMax slots: moe_sort_small_block (moe_sort.h).
__global__ __launch_bounds__(256) void moe_sort_small_kernel(const int32_t* __restrict__ ids, int S, int E,
                                                             int32_t* __restrict__ expert_offsets,
                                                             int32_t* __restrict__ sorted_slots,
                                                             int32_t* __restrict__ slot_to_pos) {
    __shared__ MoeSortSmallLds lds;
    int lo[2], hi[2];
    moe_sort_small_block(ids, S, E, blockIdx.x, true, expert_offsets, sorted_slots, slot_to_pos, lds, lo, hi);
}

// (declared in moe_common.h for the layers that launch other work in front of the routing)
int moe_topk_grouped_sigmoid_check(int T, int E, int k, int n_group, int topk_group) {
    if (T <= 0 || T > (1 << 30) || E <= 0 || k <= 0 || k > 64 || E > 64 * kMaxPerLane || n_group <= 0 || n_group > 64 ||
        (E % n_group) != 0 || topk_group <= 0 || topk_group > n_group ||
        k > topk_group * (E / n_group))
        return HK_ERR_BAD_SHAPE;
    return HK_OK;
}

}  // namespace hk

extern "C" int hk_moe_topk_softmax(const float* logits, int T, int E, int k, int32_t* ids, float* w,
                                   void* stream) {
    using namespace hk;
    if (!logits || !ids || !w) return HK_ERR_NULL_POINTER;
    if (T <= 0 || T > (1 << 30) || E <= 0 || k <= 0 || k > E || k > 64 || E > 64 * kMaxPerLane) return HK_ERR_BAD_SHAPE;
    if (E <= 128 && k <= 16)
        hipLaunchKernelGGL(moe_topk_softmax_kernel<16>, dim3((T + 15) / 16), dim3(256), 0, (hipStream_t)stream,
                           logits, T, E, k, ids, w);
    else
        hipLaunchKernelGGL(moe_topk_softmax_kernel<64>, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream,
                           logits, T, E, k, ids, w);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_topk_grouped_sigmoid(const float* logits, const float* bias_or_null, int T, int E,
                                           int k, int n_group, int topk_group, float routed_scale,
                                           int32_t* ids, float* w, void* stream) {
    using namespace hk;
    if (!logits || !ids || !w) return HK_ERR_NULL_POINTER;
    if (moe_topk_grouped_sigmoid_check(T, E, k, n_group, topk_group) != HK_OK) return HK_ERR_BAD_SHAPE;
    // 16 lanes per token when the experts split into 16 equal runs and every group is a
    // power-of-two number of whole runs
    const int per = E / 16, gs = E / n_group;
    const int lanes_per_group = per > 0 && (E % 16) == 0 && (gs % per) == 0 ? gs / per : 0;
    int lg_shift = -1;
    for (int q = 0; q <= 4; ++q)
        if (lanes_per_group == (1 << q)) lg_shift = q;
    if (lg_shift >= 0 && k <= 16 && (per == 4 || per == 8 || per == 12 || per == 16)) {
        const dim3 grid((T + 15) / 16), block(256);
        hipStream_t s = (hipStream_t)stream;
        switch (per) {
            case 4: hipLaunchKernelGGL(moe_topk_grouped_sigmoid16_kernel<4>, grid, block, 0, s, logits, bias_or_null, T, k, lg_shift, topk_group, routed_scale, ids, w); break;
            case 8: hipLaunchKernelGGL(moe_topk_grouped_sigmoid16_kernel<8>, grid, block, 0, s, logits, bias_or_null, T, k, lg_shift, topk_group, routed_scale, ids, w); break;
            case 12: hipLaunchKernelGGL(moe_topk_grouped_sigmoid16_kernel<12>, grid, block, 0, s, logits, bias_or_null, T, k, lg_shift, topk_group, routed_scale, ids, w); break;
            default: hipLaunchKernelGGL(moe_topk_grouped_sigmoid16_kernel<16>, grid, block, 0, s, logits, bias_or_null, T, k, lg_shift, topk_group, routed_scale, ids, w); break;
        }
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(moe_topk_grouped_sigmoid_kernel, dim3((T + 3) / 4), dim3(256), 0,
                       (hipStream_t)stream, logits, bias_or_null, T, E, k, n_group, topk_group,
                       routed_scale, ids, w);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" size_t hk_moe_sort_workspace_bytes(int T, int k, int E) {
    if (T <= 0 || k <= 0 || E <= 0) return 0;
    const size_t S = (size_t)T * k;
    const size_t nchunks = (S + hk::kSortChunk - 1) / hk::kSortChunk;
    return (nchunks + 1) * (size_t)E * sizeof(int32_t);  // per-chunk counts + per-expert totals
}

extern "C" int hk_moe_sort(const int32_t* ids, int T, int k, int E, int32_t* sorted_slots,
                           int32_t* expert_offsets, int32_t* slot_to_pos_or_null, void* workspace,
                           size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (!ids || !sorted_slots || !expert_offsets) return HK_ERR_NULL_POINTER;
    // (2^30 slots: the kernels index slots and chunk ends with ints)
    if (T <= 0 || k <= 0 || E <= 0 || E > kSortMaxE || (long long)T * k > (1ll << 30)) return HK_ERR_BAD_SHAPE;
    if (!workspace || workspace_bytes < hk_moe_sort_workspace_bytes(T, k, E)) return HK_ERR_WORKSPACE;
    const int S = T * k;
    const int nchunks = (S + kSortChunk - 1) / kSortChunk;
    hipStream_t s = (hipStream_t)stream;
    if (S <= kSortSmallMax) {
        hipLaunchKernelGGL(moe_sort_small_kernel, dim3(nchunks), dim3(256), 0, s, ids, S, E, expert_offsets,
                           sorted_slots, slot_to_pos_or_null);
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    int32_t* ws = (int32_t*)workspace;
    hipLaunchKernelGGL(moe_sort_count_kernel, dim3(nchunks), dim3(256), 0, s, ids, S, E, ws);
    if (nchunks <= kSortFusedChunks) {
        hipLaunchKernelGGL(moe_sort_scan_offsets_kernel, dim3(1), dim3(512), 0, s, ws, nchunks, E, expert_offsets);
        hipLaunchKernelGGL(moe_sort_scatter_kernel, dim3(nchunks), dim3(256), 0, s, ids, S, E,
                           (const int32_t*)ws, (const int32_t*)expert_offsets, sorted_slots, slot_to_pos_or_null);
    } else {
        int32_t* totals = ws + (size_t)nchunks * E;
        hipLaunchKernelGGL(moe_sort_scan_kernel, dim3(E), dim3(256), 0, s, ws, nchunks, E, totals);
        hipLaunchKernelGGL(moe_sort_scatter_totals_kernel, dim3(nchunks), dim3(256), 0, s, ids, S, E,
                           (const int32_t*)ws, (const int32_t*)totals, expert_offsets, sorted_slots,
                           slot_to_pos_or_null);
    }
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}
