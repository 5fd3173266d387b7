// Score tables for the one-pass backward of windows of 161 .. 256 tokens (fwa2_bwd_one.hip): (bias + mask) * log2e
// in fp32, in the order in which the 16 x 16 score accumulators of a wavefront hold a block of 32 queries, so that
// the backward loads a block's values straight into the C operand of its score products and bias and mask never
// pass through the VALU there.
//
// Takes the place of the bias / mask loads inside the reference's _bwd_kernel
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:222-245).
#include "fwa2_common.hpp"

namespace fwa2 {

constexpr int kTableRows = 256;     // padded rows (queries and keys) of a unit
constexpr int kTableBlocks = 8;     // query blocks of 32
constexpr int kTableLive = 256;     // windows whose mask flags the backward lists (more: every window counts as live)

// tab[slot][key tile j][query block qb][t][lane][i] = (bias[h][q][key] + mask[w][q][key]) * log2e with key = 16 j +
// lane % 16 and q = 32 qb + 8 (lane / 16) + 4 t + i; -inf for padded keys, 0 for padded queries.  Slot h < heads: the
// bias of head h alone; slot heads + w * heads + h: with the mask of window w (built only for windows whose mask is
// live; every window without flags).  One workgroup per (query block, slot): the 32 rows are read a row at a time
// (consecutive lanes, consecutive keys), summed into an LDS tile, and written out in table order, 16 bytes a lane.
template <class E, class ME>
__global__ void __launch_bounds__(256) build_table_kernel(const E* bias, int64_t bias_sh, int64_t bias_sn, const ME* mask,
                                                          int64_t mask_sw, int64_t mask_sn, const uint8_t* live, int n,
                                                          int heads, float* tab) {
    __shared__ float tile[32][kTableRows + 1];
    const int slot = blockIdx.y, qb = blockIdx.x;
    int h = slot, wnd = -1;
    if (slot >= heads) {
        wnd = (slot - heads) / heads;
        h = (slot - heads) - wnd * heads;
        if (live && !live[wnd]) return;
    }
    const int key = threadIdx.x;
    const E* bcol = bias ? bias + h * bias_sh + key : nullptr;
    const ME* mcol = wnd >= 0 ? mask + wnd * mask_sw + key : nullptr;
#pragma unroll 8
    for (int r = 0; r < 32; r++) {
        const int q = 32 * qb + r;
        float x = 0.f;
        if (key >= n) {
            x = -INFINITY;
        } else if (q < n) {
            if (bcol) x = (float)bcol[(int64_t)q * bias_sn];
            if (mcol) x += (float)mcol[(int64_t)q * mask_sn];
            x *= kLog2e;
        }
        tile[r][key] = x;
    }
    __syncthreads();
    float* dst = tab + (int64_t)slot * (kTableRows * kTableRows);
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int idx = it * 256 + threadIdx.x;          // (j, t, lane)
        const int lane = idx & 63, t = (idx >> 6) & 1, j = idx >> 7;
        const int col = 16 * j + (lane & 15), r0 = 8 * (lane >> 4) + 4 * t;
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = tile[r0 + i][col];
        *reinterpret_cast<f32x4*>(dst + ((int64_t)((j * kTableBlocks + qb) * 2 + t) * 64 + lane) * 4) = v;
    }
}

template <int DT>
static hipError_t build_tables(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    typedef typename Elem<DT>::E E;
    const bool masked = mask_dt >= 0;
    const bool has_tab = has_bias || masked || p.n < kTableRows;
    if (!has_tab) return hipSuccess;
    const int slots = p.heads * (1 + (masked ? p.n_windows : 0));
    const dim3 gr(kTableBlocks, slots);
    float* tab = const_cast<float*>(p.tab);
    const E* bias = has_bias ? reinterpret_cast<const E*>(p.bias) : nullptr;
    // The backward lists the flags of up to kTableLive windows; with more it treats every window as live and reads
    // every window's table, so every table has to be built then, whatever the flags say.
    const uint8_t* live = p.n_windows <= kTableLive ? p.mask_live : nullptr;
    if (mask_dt == FWA2_F32)
        hipLaunchKernelGGL((build_table_kernel<E, float>), gr, dim3(256), 0, st, bias, p.bias_sh, p.bias_sn,
                           reinterpret_cast<const float*>(p.mask), p.mask_sw, p.mask_sn, live, p.n, p.heads, tab);
    else
        hipLaunchKernelGGL((build_table_kernel<E, E>), gr, dim3(256), 0, st, bias, p.bias_sh, p.bias_sn,
                           reinterpret_cast<const E*>(p.mask), p.mask_sw, p.mask_sn, live, p.n, p.heads, tab);
    return hipGetLastError();
}

// The score tables of a call: slot h for every head, slot heads + w * heads + h for every window whose mask is live;
// p.tab points at room for heads * (1 + windows) tables of 256 x 256 floats.
hipError_t launch_score_tables(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    return dtype == FWA2_BF16 ? build_tables<FWA2_BF16>(p, has_bias, mask_dt, st) : build_tables<FWA2_F16>(p, has_bias, mask_dt, st);
}

}  // namespace fwa2
