// Pieces shared by the MoE kernels (MXFP4 and FP8 block-scaled): work items, the mapping of
// weight rows to LDS rows of the B tile, and host helpers implemented in moe_mxfp4.hip.
#pragma once
#include "gemm_tile.h"
#include "hk_host.h"

namespace hk {

// Row of the expert's weight matrix held by LDS row R (0..255) of the B tile of n-tile `n_tile`.
// mode 0 (gate+up, N = I): each wave's 64 rows alternate 16 gate rows / 16 up rows of the same 16
// h columns, permuted so that a lane ends up with 8 consecutive h columns; mode 1 (down, N = H):
// b_row_to_col permutation (8 consecutive output columns per lane).
// `interleaved` (mode 0): the caller's matrix has gate / up of h column c in rows 2c / 2c + 1
// instead of rows c / N + c.
__device__ __forceinline__ int moe_b_row(int mode, int R, int n_tile, int N, bool interleaved = false) {
    if (mode == 1) return min(n_tile * 256 + b_row_to_col(R), N - 1);
    const int wn = R >> 6, t = (R >> 4) & 3, r = R & 15;
    const int hcol = min(n_tile * 128 + 32 * wn + 8 * (r >> 2) + 4 * (t >> 1) + (r & 3), N - 1);
    return interleaved ? 2 * hcol + (t & 1) : (t & 1) * N + hcol;
}

// Work items. A work item is (m-tile, n-tile): up to kMoeBM (weight-streaming MXFP4 kernel: 192)
// consecutive sorted rows of one expert
// times one tile of weight rows. Items are listed expert by expert, n-tile by n-tile, the m-tiles
// of one (expert, n-tile) next to each other.
constexpr int kMoeBM = 128;
struct MoeItem { int expert, row_start, rows, n_tile; };

// SiLU(g) * u of the gate+up epilogues: g / (1 + exp(-g)) with the hardware exp2 and reciprocal
// (about 1 ulp each; every grouped GEMM kernel of the two MoE layers uses this same sequence, which
// is what keeps their results bit-identical to one another).
__device__ __forceinline__ float silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

inline int moe_round_up(int x, int m) { return (x + m - 1) / m * m; }
// Whether most experts' rows fit one work item of `bm` rows: mean + one standard deviation of the rows
// per expert when T * k slots spread uniformly over E experts. (The streaming kernels then read every
// weight byte once and load the weights with the non-temporal hint.)
inline bool moe_rows_fit_one_item(int T, int k, int E, int bm) {
    const double mu = (double)T * k / E;
    return mu + __builtin_sqrt(mu) <= bm;
}
// (A layer's workspace needs no room behind its last region: every fetch of activation rows, row scales and
// slot ids in the grouped GEMMs goes through a buffer descriptor that ends where its region ends, or through
// an index clamped to the region, so the piecewise fetches of a layer's last work item read zeros, not memory
// behind the region.)
// Number of CUs of the current device (cached per device ordinal).
int moe_num_compute_units();
// Shape check of hk_moe_topk_grouped_sigmoid (moe_routing.hip), for entry points that launch other work in
// front of the routing: HK_OK or HK_ERR_BAD_SHAPE.
int moe_topk_grouped_sigmoid_check(int T, int E, int k, int n_group, int topk_group);
// Item lists of the two grouped GEMMs of a layer from expert_offsets [E+1], m-tiles of up to `bm`
// rows: items1 / num_items[0] for n_tiles_n1 tiles of weight rows, items2 / num_items[1] for
// n_tiles_n2 (one launch).
void moe_launch_build_items(const int32_t* expert_offsets, int E, int bm, int n_tiles_n1, MoeItem* items1,
                            int n_tiles_n2, MoeItem* items2, int32_t* num_items, hipStream_t s);

}  // namespace hk
