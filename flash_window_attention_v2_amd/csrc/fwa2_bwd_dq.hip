// Backward, query side: dq (and the per-row terms of dlogit_scale) for gfx950.
//
// Together with fwa2_bwd.hip this replaces _bwd_preprocess_do_o_dot and
// _bwd_kernel of the reference
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:6-51, 84-564).  The
// reference adds every key block's dq contribution into an fp32 buffer with
// global atomics (:314); here one wavefront owns 32 query rows, walks over all
// keys and keeps dq_hat in its accumulators, so dq is written once, in the
// input dtype, with no atomics and no fp32 staging buffer.
//
// The structure mirrors the forward kernel: scores are computed transposed
// (rows = keys, columns = queries, v_mfma_f32_32x32x16) so that the
// accumulators of dZ^T = P^T (dP^T - delta), rounded to the input dtype, are
// directly the B operand (k = keys) of dQ_hat^T += K_hat^T dZ^T; K_hat^T comes
// out of row-major K_hat in LDS with ds_read_b64_tr_b16.  P is recomputed from
// the saved log-sum-exp; delta = rowsum(o * dO) is recomputed per query row.
//
// dq = s (dq_hat - q_hat (dq_hat . q_hat)) / |q| goes back through the
// normalisation in registers; q_hat . dq_hat summed over rows is the logit-scale
// gradient, because sum_j dC_ij c_ij = q_hat_i . dq_hat_i.
#include "fwa2_common.hpp"

namespace fwa2 {

template <int DT, bool HAS_BIAS, int MASK_DT, bool VEC>
__global__ void __launch_bounds__(512) bwd_dq_kernel(const BwdParams p) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    // q_hat and k_hat in the score type of the forward kernel (fp16 also for bf16 inputs): the recomputed scores
    // then round as the forward's did; dZ takes the same type, its partner in the dQ product being k_hat
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int N = p.n;
    const int chunk_rows = (min(N, kKeyChunk) + 63) & ~63;
    SE* Ks = reinterpret_cast<SE*>(smem_raw);
    E* Vs = reinterpret_cast<E*>(Ks + chunk_rows * kLdsStride);
    float* red = reinterpret_cast<float*>(Vs + chunk_rows * kLdsStride);   // [8]

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;       // query column of this lane
    const int hf = lane >> 5;        // which half of the k-slots / rows
    const int li = lane & 15;        // lane inside its 16-lane block (transpose reads)
    const int blk1 = (lane >> 4) & 1;

    // Workgroups go to the 8 XCDs in turn, each with an L2 of its own; a group of 8 consecutive workgroups (one per
    // XCD) does one kind of work.
    //  - Some groups sum the fp32 dk / dv partials of the key-side kernel (bound by HBM, while the dq work is bound by
    //    compute).  They are spread evenly among the others: with D dq groups out of T, group g does dq work iff
    //    floor((g + 1) D / T) > floor(g D / T), as dq group floor(g D / T).
    //  - dq group j on XCD x takes query chunk j % chunks of unit (j / chunks) * 8 + x: the chunks of one unit run on
    //    one XCD, which fetches the unit's K and V once for all of them; and the units run head by head, so that the
    //    workgroups in flight share one head's bias rows in the L2s.
    const int xcd = blockIdx.x & 7;
    int64_t j = blockIdx.x >> 3;
    if (p.dkv_blocks > 0) {
        const int64_t total = gridDim.x >> 3, dq_groups = total - p.dkv_blocks;
        const int64_t before = j * dq_groups / total, upto = (j + 1) * dq_groups / total;
        if (upto == before) {
            dkv_reduce_rows<DT>(p, (j - before) * 8 + xcd, (int)blockDim.x, (int)threadIdx.x);
            return;
        }
        j = before;
    }
    const int qc = (int)(j % p.dq_chunks);
    const int64_t unit = (j / p.dq_chunks) * 8 + xcd;
    if (unit >= (int64_t)p.bw * p.heads) return;
    const int h = (int)(unit / p.bw);
    const int b = (int)(unit - (int64_t)h * p.bw);

    // rows are addressed through the window map when there is one (cyclic shift + window partition done here)
    const E* qptr = reinterpret_cast<const E*>(p.q.ptr) + unit_off_any(p.q, p.map, b, h);
    const E* kptr = reinterpret_cast<const E*>(p.k.ptr) + unit_off_any(p.k, p.map, b, h);
    const E* vptr = reinterpret_cast<const E*>(p.v.ptr) + unit_off_any(p.v, p.map, b, h);
    const E* optr = reinterpret_cast<const E*>(p.o.ptr) + unit_off_any(p.o, p.map, b, h);
    const E* doptr = reinterpret_cast<const E*>(p.d_o.ptr) + unit_off_any(p.d_o, p.map, b, h);
    E* dqptr = reinterpret_cast<E*>(const_cast<void*>(p.dq.ptr)) + unit_off_any(p.dq, p.map, b, h);

    float s_true;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        s_true = expf(fminf(ls, kLn100));
    } else {
        s_true = p.default_scale;
    }
    const float scale2 = s_true * kLog2e;

    const int q0 = (qc * p.dq_waves + wave) * 32;
    const int qi = q0 + col;
    const bool qv = qi < N;
    const bool wave_live = q0 < N;

    // ---- per-query operands: q_hat * s * log2e, dO (both as B operands), delta, lse ----
    SV8 bq0 = zero8<SV8>(), bq1 = zero8<SV8>();
    V8 bd0 = zero8<V8>(), bd1 = zero8<V8>();
    float nlse2 = -INFINITY, ndelta = 0.f;
    if (wave_live) {
        V8 a = zero8<V8>(), c = zero8<V8>(), o0 = zero8<V8>(), o1 = zero8<V8>();
        if (qv) {
            const int qpos = unit_row_any(p.map, b, qi);
            const E* qrow = qptr + (int64_t)qpos * p.q.sn;
            const E* dorow = doptr + (int64_t)qpos * p.d_o.sn;
            const E* orow = optr + (int64_t)qpos * p.o.sn;
            a = ld8<V8>(qrow + 8 * hf);
            c = ld8<V8>(qrow + 16 + 8 * hf);
            bd0 = ld8<V8>(dorow + 8 * hf);
            bd1 = ld8<V8>(dorow + 16 + 8 * hf);
            o0 = ld8<V8>(orow + 8 * hf);
            o1 = ld8<V8>(orow + 16 + 8 * hf);
            const float l = p.lse[b * p.lse_sb + h * p.lse_sh + qi];
            nlse2 = (l == -INFINITY) ? -INFINITY : -l * kLog2e;   // fully masked row: P = 0
        }
        float xa[8], xc[8];
        unpack8(a, xa);
        unpack8(c, xc);
        float ss = 0.f, dl = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            ss += xa[j] * xa[j] + xc[j] * xc[j];
            dl += (float)o0[j] * (float)bd0[j] + (float)o1[j] * (float)bd1[j];
        }
        ss = xor32_add(ss);
        ndelta = -xor32_add(dl);
        const float sc = scale2 * inv_norm(ss);
#pragma unroll
        for (int j = 0; j < 8; j++) { bq0[j] = (SE)(xa[j] * sc); bq1[j] = (SE)(xc[j] * sc); }
    }

    const E* bias_row = nullptr;
    if (HAS_BIAS) bias_row = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)min(qi, N - 1) * p.bias_sn;
    const ME* mask_row = nullptr;
    bool mask_on = false;
    if (MASK_DT >= 0) {
        const int w = b % p.n_windows;
        mask_on = p.mask_live ? (p.mask_live[w] != 0) : true;
        mask_row = reinterpret_cast<const ME*>(p.mask) + w * p.mask_sw + (int64_t)min(qi, N - 1) * p.mask_sn;
    }

    f32x16 dqacc;
#pragma unroll
    for (int i = 0; i < 16; i++) dqacc[i] = 0.f;

    for (int c0 = 0; c0 < N; c0 += kKeyChunk) {
        const int rows = min(N - c0, kKeyChunk);
        const int rows_pad = (rows + 63) & ~63;
        if (c0 > 0) __syncthreads();
        // ---- stage K_hat and V rows c0 .. c0+rows_pad of this (b, h) ----
        for (int r = tid >> 2; r < rows_pad; r += nthreads >> 2) {
            const int dch = (tid & 3) * 8;
            V8 kk = zero8<V8>(), vv = zero8<V8>();
            if (r < rows) {
                const int pos = unit_row_any(p.map, b, c0 + r);
                kk = ld8<V8>(kptr + (int64_t)pos * p.k.sn + dch);
                vv = ld8<V8>(vptr + (int64_t)pos * p.v.sn + dch);
            }
            float x[8];
            unpack8(kk, x);
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) ss += x[j] * x[j];
            ss = quad_add(ss);
            const float inv = inv_norm(ss);
            SV8 kn;
#pragma unroll
            for (int j = 0; j < 8; j++) kn[j] = (SE)(x[j] * inv);
            st8<SV8>(Ks + r * kLdsStride + dch, kn);
            st8<V8>(Vs + r * kLdsStride + dch, vv);
        }
        __syncthreads();
        if (!wave_live) continue;

        // one 32-key tile at a time (P needs no running maximum here, the log-sum-exp is known)
        const int ntile = rows_pad >> 5;
        for (int kt = 0; kt < ntile; kt++) {
            const int kbase = c0 + kt * 32;
            // register i <-> key kbase + 16(i/8) + 8hf + i%8
            const int row = (kt * 32 + swap_bits23(col)) * kLdsStride + 8 * hf;
            const SV8 k0 = ld8<SV8>(Ks + row), k1 = ld8<SV8>(Ks + row + 16);
            const V8 v0 = ld8<V8>(Vs + row), v1 = ld8<V8>(Vs + row + 16);
            f32x16 sacc, pacc;
#pragma unroll
            for (int i = 0; i < 16; i++) { sacc[i] = nlse2; pacc[i] = ndelta; }
            sacc = Elem<kScoreDT>::mfma32(k0, bq0, sacc);
            sacc = Elem<kScoreDT>::mfma32(k1, bq1, sacc);      // (S - lse) * log2e
            pacc = Elem<DT>::mfma32(v0, bd0, pacc);
            pacc = Elem<DT>::mfma32(v1, bd1, pacc);      // dP - delta
            if (HAS_BIAS) {
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    float x[8];
                    load_row8<VEC, E>(bias_row, kbase + 16 * u + 8 * hf, N, x);
#pragma unroll
                    for (int j = 0; j < 8; j++) sacc[8 * u + j] = fmaf(x[j], kLog2e, sacc[8 * u + j]);
                }
            }
            if (MASK_DT >= 0) {
                if (mask_on) {
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        float x[8];
                        load_row8<VEC, ME>(mask_row, kbase + 16 * u + 8 * hf, N, x);
#pragma unroll
                        for (int j = 0; j < 8; j++) sacc[8 * u + j] = fmaf(x[j], kLog2e, sacc[8 * u + j]);
                    }
                }
            }
            if (kbase + 32 > N) {   // padded key columns never take part
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = kbase + 16 * (i >> 3) + 8 * hf + (i & 7);
                    if (key >= N) sacc[i] = -INFINITY;
                }
            }
            // ---- dZ^T = P^T (dP^T - delta); dQ_hat^T += K_hat^T dZ^T, 16 keys per MFMA ----
#pragma unroll
            for (int mm = 0; mm < 2; mm++) {
                SV8 bz;
#pragma unroll
                for (int j = 0; j < 8; j++) bz[j] = (SE)(fast_exp2(sacc[8 * mm + j]) * pacc[8 * mm + j]);
                const SE* klo = Ks + (kt * 32 + 16 * mm + 8 * hf + (li >> 2)) * kLdsStride + 16 * blk1 + 4 * (li & 3);
                const SV8 ak = lds_tr8<kScoreDT>(klo, klo + 4 * kLdsStride);
                dqacc = Elem<kScoreDT>::mfma32(ak, bz, dqacc);
            }
        }
    }

    // ---- back through q / max(|q|, eps): lane (query, hf) holds d = 8c + 4hf + j ----
    float dot = 0.f;
    if (wave_live) {
        float x[16];
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            V4 q4;
#pragma unroll
            for (int j = 0; j < 4; j++) q4[j] = 0;
            if (qv) q4 = *reinterpret_cast<const V4*>(qptr + (int64_t)unit_row_any(p.map, b, qi) * p.q.sn + 8 * c + 4 * hf);
#pragma unroll
            for (int j = 0; j < 4; j++) { x[4 * c + j] = (float)q4[j]; ss += x[4 * c + j] * x[4 * c + j]; }
        }
        ss = xor32_add(ss);
        const float nrm = sqrtf(ss);
        const float inv = 1.0f / fmaxf(nrm, kNormEps);
#pragma unroll
        for (int i = 0; i < 16; i++) { x[i] *= inv; dot += dqacc[i] * x[i]; }
        dot = xor32_add(dot);
        const float proj = nrm > kNormEps ? dot : 0.f;
        const float f = s_true * inv;
        if (qv) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                V4 o4;
#pragma unroll
                for (int j = 0; j < 4; j++) o4[j] = (E)(f * (dqacc[4 * c + j] - x[4 * c + j] * proj));
                *reinterpret_cast<V4*>(dqptr + (int64_t)unit_row_any(p.map, b, qi) * p.dq.sn + 8 * c + 4 * hf) = o4;
            }
        }
        if (!qv || hf != 0) dot = 0.f;
    }
    // ---- dlogit_scale: one partial per workgroup ----
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float wsum = wave_sum(dot);
        __syncthreads();
        if (lane == 0) red[wave] = wsum;
        __syncthreads();
        if (tid == 0) {
            float tot = 0.f;
            for (int i = 0; i < p.dq_waves; i++) tot += red[i];
            p.part_dscale[(int64_t)h * p.ds_parts + (int64_t)b * p.dq_chunks + qc] = tot * s_true;
        }
    }
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_one(const BwdParams& p, dim3 grid, dim3 block, size_t smem, hipStream_t st) {
    if (p.side_vec)
        hipLaunchKernelGGL((bwd_dq_kernel<DT, HAS_BIAS, MASK_DT, true>), grid, block, smem, st, p);
    else
        hipLaunchKernelGGL((bwd_dq_kernel<DT, HAS_BIAS, MASK_DT, false>), grid, block, smem, st, p);
    return hipGetLastError();
}

template <int DT>
static hipError_t launch_dt(const BwdParams& p, bool has_bias, int mask_dt, dim3 g, dim3 b, size_t s, hipStream_t st) {
    if (has_bias) {
        if (mask_dt < 0) return launch_one<DT, true, -1>(p, g, b, s, st);
        if (mask_dt == FWA2_F32) return launch_one<DT, true, FWA2_F32>(p, g, b, s, st);
        return launch_one<DT, true, DT>(p, g, b, s, st);
    }
    if (mask_dt < 0) return launch_one<DT, false, -1>(p, g, b, s, st);
    if (mask_dt == FWA2_F32) return launch_one<DT, false, FWA2_F32>(p, g, b, s, st);
    return launch_one<DT, false, DT>(p, g, b, s, st);
}

// Wavefronts per workgroup and workgroups per (batch*window, head) of the dq kernel.
void dq_geometry(int n, int* waves, int* chunks) {
    const int q_tiles = (n + 31) / 32;
    *waves = q_tiles < 8 ? q_tiles : 8;
    *chunks = (q_tiles + *waves - 1) / *waves;
}

hipError_t launch_backward_dq(const BwdParams& p_in, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    BwdParams p = p_in;
    const int chunk_rows = ((p.n < kKeyChunk ? p.n : kKeyChunk) + 63) & ~63;
    const size_t smem = (size_t)2 * chunk_rows * kLdsStride * 2 + 8 * sizeof(float);
    const dim3 block(64 * p.dq_waves);
    // groups of 8 workgroups: dq groups cover (unit, chunk) for the units rounded up to a multiple of 8 ...
    const int64_t dq_groups = (((int64_t)p.bw * p.heads + 7) / 8) * p.dq_chunks;
    // ... and the fp32 dk / dv partials of the super-tiled key-side kernel are summed by extra groups of this launch
    const int64_t rows_per_block = block.x / 4, rows = (int64_t)p.bw * p.heads * p.n;
    const int64_t dkv_blocks = p.n_chunks > 1 ? (rows + rows_per_block - 1) / rows_per_block : 0;
    p.dkv_blocks = (int)((dkv_blocks + 7) / 8);        // (counted in groups)
    if ((dq_groups + p.dkv_blocks) * 8 > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)((dq_groups + p.dkv_blocks) * 8));
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, grid, block, smem, st);
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, grid, block, smem, st);
}

}  // namespace fwa2
