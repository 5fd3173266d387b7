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
// live; every window without flags).  One thread per 16 bytes of table: eight independent 2-byte loads (16 lanes read
// 32 consecutive bytes of a row), one 16-byte store.  (A form that reads whole rows through an LDS tile, one workgroup
// per query block and slot, has too few workgroups in flight and measured twice as slow.)
template <class E, class ME>
__global__ void __launch_bounds__(256) build_table_kernel(const E* bias, int64_t bias_sh, int64_t bias_sn, const ME* mask,
                                                          int64_t mask_sw, int64_t mask_sn, const uint8_t* live, int n,
                                                          int heads, float* tab) {
    const int slot = blockIdx.y;
    int h = slot, wnd = -1;
    if (slot >= heads) {
        wnd = (slot - heads) / heads;
        h = (slot - heads) - wnd * heads;
        if (live && !live[wnd]) return;
    }
    const int idx = blockIdx.x * 256 + threadIdx.x;        // (j, qb, t, lane)
    const int lane = idx & 63, t = (idx >> 6) & 1, rest = idx >> 7;
    const int qb = rest % kTableBlocks, j = rest / kTableBlocks;
    const int key = 16 * j + (lane & 15), q0 = 32 * qb + 8 * (lane >> 4) + 4 * t;
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int q = q0 + i;
        float x = 0.f;
        if (key >= n) {
            x = -INFINITY;
        } else if (q < n) {
            if (bias) x = (float)bias[h * bias_sh + (int64_t)q * bias_sn + key];
            if (wnd >= 0) x += (float)mask[wnd * mask_sw + (int64_t)q * mask_sn + key];
            x *= kLog2e;
        }
        v[i] = x;
    }
    *reinterpret_cast<f32x4*>(tab + (int64_t)slot * (kTableRows * kTableRows) + (int64_t)idx * 4) = v;
}

template <int DT>
static hipError_t build_tables(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    typedef typename Elem<DT>::E E;
    const bool masked = mask_dt >= 0;
    const bool has_tab = has_bias || masked || p.n < kTableRows;
    if (!has_tab) return hipSuccess;
    const int slots = p.heads * (1 + (masked ? p.n_windows : 0));
    const dim3 gr(kTableRows * kTableRows / 4 / 256, slots);
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
