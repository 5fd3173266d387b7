// Forward kernel: o, lse = softmax(s * q_hat k_hat^T + bias + mask) v  for gfx950.
//
// Replaces the Triton kernel _fwd_kernel of the reference
// (flash_win_attn_v2/kernels/attn_kernel_forward.py:33-258).
//
// Work split.  One workgroup owns one (batch*window, head) pair and a chunk of
// up to 32*waves query rows; each wavefront owns 32 query rows and walks over
// all keys in blocks of 64.  K (L2-normalised, in the input dtype) and V are
// staged once per workgroup in LDS, 256 keys at a time.
//
// Matrix shapes.  Scores are computed transposed, S^T = K_hat Q_hat^T, with
// v_mfma_f32_32x32x16: rows = keys, columns = queries.  A lane then holds, for
// ONE query (column lane%32), the scores of 16 keys of the tile in its
// accumulator registers, so the softmax row reductions are in-lane plus one
// exchange with the lane 32 away, and the exponentiated accumulators are
// directly the B operand (k = keys) of the second MFMA O^T = V^T P^T.  The rows
// of each 32-key tile are permuted (swap_bits23) so that the 8 registers fed
// to one MFMA are 8 consecutive keys; V^T comes out of row-major V in LDS with
// ds_read_b64_tr_b16.
//
// Numerics.  Scores live in the log2 domain: q_hat is multiplied by
// s * log2(e) in fp32 before it is rounded to fp16 (also for bf16 inputs: the
// normalised vectors fit fp16's range and gain 3 mantissa bits), bias and mask
// are multiplied by log2(e) in fp32, exp is v_exp_f32 (2^x).  Softmax state,
// accumulators and the log-sum-exp are fp32; P is rounded to the input dtype
// for the second MFMA (as the reference does, attn_kernel_forward.py:225-226).
#include "fwa2_common.hpp"

namespace fwa2 {

template <int DT, bool HAS_BIAS, int MASK_DT, bool VEC>
__global__ void __launch_bounds__(512) fwd_kernel(const FwdParams p) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    // the cosine scores always go through the fp16 matrix path: q_hat and k_hat lie in [-1, 1]
    // (times a scale <= 100 log2 e), where fp16 keeps 3 more mantissa bits than bf16
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int N = p.n;
    const int chunk_rows = (min(N, kKeyChunk) + 63) & ~63;
    SE* Ks = reinterpret_cast<SE*>(smem_raw);
    E* Vs = reinterpret_cast<E*>(Ks + chunk_rows * kLdsStride);

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;       // query column of this lane
    const int hf = lane >> 5;        // which half of the k-slots / rows
    const int li = lane & 15;        // lane inside its 16-lane block (transpose reads)
    const int blk1 = (lane >> 4) & 1;

    // Workgroup -> (query chunk, unit).  Workgroups go to the 8 XCDs in turn, each with an L2 of its own, so the
    // chunks of one unit are given to workgroups 8 apart (one XCD fetches the unit's K and V once for all of them),
    // and the units run head by head, so that the workgroups in flight share one head's bias rows in those L2s.
    const int units = p.bw * p.heads, units8 = units & ~7;
    int qc, unit;
    if ((int)blockIdx.x < units8 * p.q_chunks) {
        const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
        qc = j % p.q_chunks;
        unit = (j / p.q_chunks) * 8 + xcd;
    } else {
        const int r = blockIdx.x - units8 * p.q_chunks;
        qc = r % p.q_chunks;
        unit = units8 + r / p.q_chunks;
    }
    const int h = unit / p.bw;
    const int b = unit - h * p.bw;

    // rows are addressed through the window map when there is one (cyclic shift + window partition done here)
    const E* qptr = reinterpret_cast<const E*>(p.q.ptr) + unit_off_any(p.q, p.map, b, h);
    const E* kptr = reinterpret_cast<const E*>(p.k.ptr) + unit_off_any(p.k, p.map, b, h);
    const E* vptr = reinterpret_cast<const E*>(p.v.ptr) + unit_off_any(p.v, p.map, b, h);
    E* optr = reinterpret_cast<E*>(const_cast<void*>(p.o.ptr)) + unit_off_any(p.o, p.map, b, h);

    float scale2;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        scale2 = expf(fminf(ls, kLn100)) * kLog2e;
    } else {
        scale2 = p.default_scale * kLog2e;
    }

    const int q0 = (qc * p.waves + wave) * 32;
    const int qi = q0 + col;
    const bool qv = qi < N;
    const bool wave_live = q0 < N;

    // ---- Q operand: normalise, fold the scale, round to the input dtype ----
    SV8 bq0 = zero8<SV8>(), bq1 = zero8<SV8>();
    if (wave_live) {
        V8 a = zero8<V8>(), c = zero8<V8>();
        if (qv) {
            const E* qrow = qptr + (int64_t)unit_row_any(p.map, b, qi) * p.q.sn;
            a = ld8<V8>(qrow + 8 * hf);
            c = ld8<V8>(qrow + 16 + 8 * hf);
        }
        float xa[8], xc[8];
        unpack8(a, xa);
        unpack8(c, xc);
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) ss += xa[j] * xa[j] + xc[j] * xc[j];
        ss = xor32_add(ss);
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

    float m_run = -INFINITY;   // running row max (log2 domain)
    float l_run = 0.f;         // this lane's share of the running row sum
    f32x16 oacc;
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[i] = 0.f;

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

        const int nblk = rows_pad >> 6;
        for (int kb = 0; kb < nblk; kb++) {
            // ---- S^T tiles: 2 x (32 keys x 32 queries) ----
            f32x16 acc[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const SE* krow = Ks + (kb * 64 + 32 * t + swap_bits23(col)) * kLdsStride + 8 * hf;
                SV8 a0 = ld8<SV8>(krow);
                SV8 a1 = ld8<SV8>(krow + 16);
                f32x16 z;
#pragma unroll
                for (int i = 0; i < 16; i++) z[i] = 0.f;
                z = Elem<kScoreDT>::mfma32(a0, bq0, z);
                acc[t] = Elem<kScoreDT>::mfma32(a1, bq1, z);
            }
            // register i of tile t <-> key kbase + 32t + 16(i/8) + 8hf + i%8
            const int kbase = c0 + kb * 64;
            if (HAS_BIAS) {
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        float x[8];
                        load_row8<VEC, E>(bias_row, kbase + 32 * t + 16 * u + 8 * hf, N, x);
#pragma unroll
                        for (int j = 0; j < 8; j++) acc[t][8 * u + j] = fmaf(x[j], kLog2e, acc[t][8 * u + j]);
                    }
            }
            if (MASK_DT >= 0) {
                if (mask_on) {
#pragma unroll
                    for (int t = 0; t < 2; t++)
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            float x[8];
                            load_row8<VEC, ME>(mask_row, kbase + 32 * t + 16 * u + 8 * hf, N, x);
#pragma unroll
                            for (int j = 0; j < 8; j++) acc[t][8 * u + j] = fmaf(x[j], kLog2e, acc[t][8 * u + j]);
                        }
                }
            }
            if (kbase + 64 > N) {   // padded key columns never take part
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int key = kbase + 32 * t + 16 * (i >> 3) + 8 * hf + (i & 7);
                        if (key >= N) acc[t][i] = -INFINITY;
                    }
            }
            // ---- online softmax over this 64-key block ----
            float bm = acc[0][0];
#pragma unroll
            for (int i = 1; i < 16; i++) bm = fmaxf(bm, acc[0][i]);
#pragma unroll
            for (int i = 0; i < 16; i++) bm = fmaxf(bm, acc[1][i]);
            bm = xor32_max(bm);
            const float m_new = fmaxf(m_run, bm);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_use);
            m_run = m_new;
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    acc[t][i] = fast_exp2(acc[t][i] - m_use);
                    psum += acc[t][i];
                }
            l_run = l_run * alpha + psum;
#pragma unroll
            for (int i = 0; i < 16; i++) oacc[i] *= alpha;
            // ---- O^T += V^T P^T, 16 keys per MFMA ----
#pragma unroll
            for (int mm = 0; mm < 4; mm++) {
                V8 bp;
#pragma unroll
                for (int j = 0; j < 8; j++) bp[j] = (E)acc[mm >> 1][8 * (mm & 1) + j];
                const E* vlo = Vs + (kb * 64 + 16 * mm + 8 * hf + (li >> 2)) * kLdsStride + 16 * blk1 + 4 * (li & 3);
                V8 av = lds_tr8<DT>(vlo, vlo + 4 * kLdsStride);
                oacc = Elem<DT>::mfma32(av, bp, oacc);
            }
        }
    }

    if (!wave_live) return;
    // ---- normalise, write o (input dtype) and lse (natural log, fp32) ----
    const float l_tot = xor32_add(l_run);
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (qv) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            V4 ov;
#pragma unroll
            for (int j = 0; j < 4; j++) ov[j] = (E)(oacc[4 * c + j] * inv_l);
            *reinterpret_cast<V4*>(optr + (int64_t)unit_row_any(p.map, b, qi) * p.o.sn + 8 * c + 4 * hf) = ov;
        }
        if (hf == 0) {
            const float lse = l_tot > 0.f ? (m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
            p.lse[b * p.lse_sb + h * p.lse_sh + qi] = lse;
        }
    }
}

// One byte of flags per window.  0: the [N, N] mask is all zero.  Bit 0: it holds a non-zero entry.
// Bit 1 (with bit 0): no entry is positive (or NaN) and every row keeps at least one exact zero, so
// the mask can only remove keys and never removes all of a row.
// Bit 2 (with bits 0 and 1, only when `regions` is given and n <= 256): the mask is EXACTLY
// c * [id_i != id_j] for one finite c < 0 and a labelling of the tokens with at most kMaxRegions ids, which
// is what the shifted-window construction produces (swin_transformer_v2.py:386-405 of the reference: ids
// painted on the rolled grid, -100 where they differ).  The window's record in `regions` then holds c and
// the ids (RegionRecord); every entry of the mask has been compared with that form, so a kernel may rebuild
// the window's mask from the record instead of reading it.
template <class ME>
__global__ void __launch_bounds__(256) mask_scan_kernel(const ME* mask, int64_t sw, int64_t sn, int n,
                                                        uint8_t* live, uint8_t* regions) {
    const int w = blockIdx.x;
    const ME* m = mask + w * sw;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    __shared__ int lds_rep[256];          // first column of the row that holds an exact zero (n if none)
    __shared__ float lds_lo[256], lds_hi[256];
    __shared__ uint8_t lds_id[256];
    const bool want = regions != nullptr && n <= 256;
    int any = 0, unsafe = 0;
    float lo = INFINITY, hi = -INFINITY;  // range of the non-zero entries this thread saw
    for (int r = wave; r < n; r += 4) {       // one wavefront per row, coalesced along the row
        int first = n;
        for (int c = lane; c < n; c += 64) {
            const float v = (float)m[r * sn + c];
            any |= (v != 0.f);
            unsafe |= !(v <= 0.f);
            if (v == 0.f) first = min(first, c);
            else { lo = fminf(lo, v); hi = fmaxf(hi, v); }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off));
        if (first == n) unsafe = 1;
        if (want && lane == 0) lds_rep[r] = first;
    }
    any = __syncthreads_or(any);
    unsafe = __syncthreads_or(unsafe);
    uint8_t flags = any ? (unsafe ? 1 : 3) : 0;
    if (want && flags == 3) {
        // the one non-zero value
        lds_lo[tid] = lo;
        lds_hi[tid] = hi;
        __syncthreads();
        for (int off = 128; off > 0; off >>= 1) {
            if (tid < off) {
                lds_lo[tid] = fminf(lds_lo[tid], lds_lo[tid + off]);
                lds_hi[tid] = fmaxf(lds_hi[tid], lds_hi[tid + off]);
            }
            __syncthreads();
        }
        const float cval = lds_lo[0];
        int bad = !(cval == lds_hi[0]) || !(cval < 0.f) || !(cval * kLog2e > -kMaxRegionValue2);
        // tokens of a region all see their first zero at the region's smallest token: that token stands for
        // the region, and ids number the regions in the order of those tokens
        int id = 0, reps = 0;
        if (tid < n) {
            const int rep = lds_rep[tid];
            bad |= rep > tid;                            // the diagonal must be zero
            for (int j = 0; j < n; j++) {
                const int is_rep = lds_rep[j] == j;
                reps += is_rep;
                id += is_rep && j < rep;
            }
            bad |= reps > kMaxRegions;
            lds_id[tid] = (uint8_t)(id & 255);
        }
        bad = __syncthreads_or(bad);
        if (!bad) {
            // every entry against the form
            for (int r = wave; r < n; r += 4) {
                const int idr = lds_id[r];
                for (int c = lane; c < n; c += 64) {
                    const float v = (float)m[r * sn + c];
                    const float want_v = (lds_id[c] != idr) ? cval : 0.f;
                    bad |= !(v == want_v);
                }
            }
            bad = __syncthreads_or(bad);
        }
        if (!bad) {
            flags |= 4;
            RegionRecord* rec = reinterpret_cast<RegionRecord*>(regions + (size_t)w * sizeof(RegionRecord));
            if (tid == 0) { rec->value = cval; rec->count = reps; rec->pad[0] = 0; rec->pad[1] = 0; }
            rec->id[tid] = tid < n ? lds_id[tid] : 0;
        }
    }
    if (tid == 0) live[w] = flags;
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_one(const FwdParams& p, dim3 grid, dim3 block, size_t smem, hipStream_t st) {
    if (p.side_vec)
        hipLaunchKernelGGL((fwd_kernel<DT, HAS_BIAS, MASK_DT, true>), grid, block, smem, st, p);
    else
        hipLaunchKernelGGL((fwd_kernel<DT, HAS_BIAS, MASK_DT, false>), grid, block, smem, st, p);
    return hipGetLastError();
}

template <int DT>
static hipError_t launch_dt(const FwdParams& p, bool has_bias, int mask_dt, dim3 g, dim3 b, size_t s, hipStream_t st) {
    if (has_bias) {
        if (mask_dt < 0) return launch_one<DT, true, -1>(p, g, b, s, st);
        if (mask_dt == FWA2_F32) return launch_one<DT, true, FWA2_F32>(p, g, b, s, st);
        return launch_one<DT, true, DT>(p, g, b, s, st);
    }
    if (mask_dt < 0) return launch_one<DT, false, -1>(p, g, b, s, st);
    if (mask_dt == FWA2_F32) return launch_one<DT, false, FWA2_F32>(p, g, b, s, st);
    return launch_one<DT, false, DT>(p, g, b, s, st);
}

int forward_resident_supported(int n);
hipError_t launch_forward_resident(const FwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st);

hipError_t launch_forward(FwdParams p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    // windows of up to 256 tokens keep the bias tile in registers; longer ones stream it
    if (forward_resident_supported(p.n)) return launch_forward_resident(p, dtype, has_bias, mask_dt, st);
    const int q_tiles = (p.n + 31) / 32;
    p.waves = q_tiles < 8 ? q_tiles : 8;
    p.q_chunks = (q_tiles + p.waves - 1) / p.waves;
    const int chunk_rows = ((p.n < kKeyChunk ? p.n : kKeyChunk) + 63) & ~63;
    const size_t smem = (size_t)2 * chunk_rows * kLdsStride * 2;
    dim3 grid((unsigned)((int64_t)p.bw * p.heads * p.q_chunks)), block(64 * p.waves);
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, grid, block, smem, st);
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, grid, block, smem, st);
}

hipError_t launch_mask_scan(const void* mask, int mask_dt, int64_t sw, int64_t sn, int n, int n_windows,
                            uint8_t* live, uint8_t* regions, hipStream_t st) {
    dim3 grid(n_windows), block(256);
    if (mask_dt == FWA2_F32)
        hipLaunchKernelGGL(mask_scan_kernel<float>, grid, block, 0, st, (const float*)mask, sw, sn, n, live, regions);
    else if (mask_dt == FWA2_BF16)
        hipLaunchKernelGGL(mask_scan_kernel<__bf16>, grid, block, 0, st, (const __bf16*)mask, sw, sn, n, live, regions);
    else
        hipLaunchKernelGGL(mask_scan_kernel<_Float16>, grid, block, 0, st, (const _Float16*)mask, sw, sn, n, live, regions);
    return hipGetLastError();
}

}  // namespace fwa2
