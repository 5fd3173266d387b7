// Relative position bias of a window from its table, and the gradient back into table space.
//
// Replaces the tail of WindowAttention's bias path in the reference
// (flash_win_attn_v2/swin_transformer_v2.py:283-287): gather by relative_position_index,
// permute to [H, N, N], 16 * sigmoid -- and, in backward, the sigmoid derivative and the
// index_put(accumulate) of the [H, N, N] gradient into the (2Wh-1)(2Ww-1) x H table, which
// framework autograd does with a sort.  The index is the closed form
//   idx(q, k) = (r_q - r_k + Wh - 1) (2 Ww - 1) + (c_q - c_k + Ww - 1),   token = r * Ww + c,
// so entry idx of the table collects the pairs (q, k) that lie the same offset apart: the
// backward is a plain sum per table entry, in a fixed order (bit-reproducible), in fp32.
#include "fwa2_common.hpp"

namespace fwa2 {

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + __expf(-x)); }

// bias[h][q][k] = 16 * round(sigmoid(table[idx(q, k)][h]))   (rounded to the element type before the
// exact scaling by 16, as the reference's two framework calls do)
template <class E>
__global__ void __launch_bounds__(256) cpb_bias_fwd_kernel(const E* table, int heads, int wh, int ww, E* bias) {
    const int n = wh * ww;
    const int64_t total = (int64_t)heads * n * n;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int k = (int)(i % n);
    const int q = (int)((i / n) % n);
    const int h = (int)(i / ((int64_t)n * n));
    const int idx = (q / ww - k / ww + wh - 1) * (2 * ww - 1) + (q % ww - k % ww + ww - 1);
    const float s = (float)(E)sigmoidf((float)table[(int64_t)idx * heads + h]);
    bias[i] = (E)(16.0f * s);
}

// dtable[idx][h] = 16 s (1 - s) * sum over the pairs (q, k) of that offset of dbias[h][q][k].
// One 64-lane workgroup per (table entry, head); the pairs of an entry are q = (r, c) with
// max(0, dr) <= r < min(Wh, Wh + dr), likewise c, and k = (r - dr, c - dc).
template <class E>
__global__ void __launch_bounds__(64) cpb_bias_bwd_kernel(const E* table, const E* dbias, int heads, int wh, int ww,
                                                          E* dtable) {
    const int idx = blockIdx.x, h = blockIdx.y;
    const int n = wh * ww;
    const int dr = idx / (2 * ww - 1) - (wh - 1);
    const int dc = idx % (2 * ww - 1) - (ww - 1);
    const int r0 = dr > 0 ? dr : 0, r1 = dr < 0 ? wh + dr : wh;
    const int c0 = dc > 0 ? dc : 0, c1 = dc < 0 ? ww + dc : ww;
    const int nc = c1 - c0, pairs = (r1 - r0) * nc;
    const E* src = dbias + (int64_t)h * n * n;
    float acc = 0.f;
    for (int i = threadIdx.x; i < pairs; i += 64) {
        const int r = r0 + i / nc, c = c0 + i % nc;
        const int q = r * ww + c, k = (r - dr) * ww + (c - dc);
        acc += (float)src[(int64_t)q * n + k];
    }
    acc = wave_sum(acc);
    if (threadIdx.x == 0) {
        const float s = sigmoidf((float)table[(int64_t)idx * heads + h]);
        dtable[(int64_t)idx * heads + h] = (E)(16.0f * s * (1.0f - s) * acc);
    }
}

hipError_t launch_cpb_bias_forward(const void* table, int dtype, int heads, int wh, int ww, void* bias, hipStream_t st) {
    const int64_t total = (int64_t)heads * wh * ww * wh * ww;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (dtype == FWA2_BF16)
        hipLaunchKernelGGL(cpb_bias_fwd_kernel<Elem<FWA2_BF16>::E>, grid, block, 0, st,
                           reinterpret_cast<const Elem<FWA2_BF16>::E*>(table), heads, wh, ww,
                           reinterpret_cast<Elem<FWA2_BF16>::E*>(bias));
    else
        hipLaunchKernelGGL(cpb_bias_fwd_kernel<Elem<FWA2_F16>::E>, grid, block, 0, st,
                           reinterpret_cast<const Elem<FWA2_F16>::E*>(table), heads, wh, ww,
                           reinterpret_cast<Elem<FWA2_F16>::E*>(bias));
    return hipGetLastError();
}

hipError_t launch_cpb_bias_backward(const void* table, const void* dbias, int dtype, int heads, int wh, int ww,
                                    void* dtable, hipStream_t st) {
    const dim3 grid((2 * wh - 1) * (2 * ww - 1), heads), block(64);
    if (dtype == FWA2_BF16)
        hipLaunchKernelGGL(cpb_bias_bwd_kernel<Elem<FWA2_BF16>::E>, grid, block, 0, st,
                           reinterpret_cast<const Elem<FWA2_BF16>::E*>(table),
                           reinterpret_cast<const Elem<FWA2_BF16>::E*>(dbias), heads, wh, ww,
                           reinterpret_cast<Elem<FWA2_BF16>::E*>(dtable));
    else
        hipLaunchKernelGGL(cpb_bias_bwd_kernel<Elem<FWA2_F16>::E>, grid, block, 0, st,
                           reinterpret_cast<const Elem<FWA2_F16>::E*>(table),
                           reinterpret_cast<const Elem<FWA2_F16>::E*>(dbias), heads, wh, ww,
                           reinterpret_cast<Elem<FWA2_F16>::E*>(dtable));
    return hipGetLastError();
}

}  // namespace fwa2
