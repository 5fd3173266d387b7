// Forward for windows of up to 256 tokens: persistent workgroups with the bias
// tile resident in registers.
//
// Replaces _fwd_kernel (flash_win_attn_v2/kernels/attn_kernel_forward.py:33-258)
// for N <= 256; longer windows go through the streaming kernel in fwa2_fwd.hip.
//
// A workgroup belongs to one head and walks over many (batch*window) units.
// Each wavefront owns 16 query rows; for them it loads bias[h] * log2(e) once,
// in the register layout of the score accumulators, and from then on every
// score tile starts from those registers as the MFMA's C operand: the bias
// costs no instruction and no memory access in the unit loop.
//
// Cosine scores are bounded, |s q_hat.k_hat| <= s, so for a query row
// m = s log2e + max_j bias2[j] bounds every logit of the row from above and the
// largest logit is at least m - 2 s log2e (the key that holds the largest bias
// scores at least -s).  When that gap (plus the bias range, for units whose
// mask removes keys) leaves exp2 comfortably inside the fp32 / bf16 exponent
// range, m is folded into the resident registers and the softmax needs no
// running maximum at all: P~ = 2^acc, l = sum P~, o = (P~ V) / l,
// lse = (m + log2 l) ln 2.  Otherwise (fp16 P would underflow, scales near the
// clamp of 100, masks with positive entries or fully masked rows) the same
// loop runs with the usual running maximum.
//
// Per unit: K_hat (fp16) and V of the NEXT unit are fetched into registers
// before the tiles of the current one are computed, normalised and written to
// the other half of a double buffer afterwards; one barrier per unit.
#include "fwa2_common.hpp"

namespace fwa2 {

constexpr float kGapLimit = 96.f;   // largest tolerated (row bound - largest logit), log2 domain

__device__ __forceinline__ float xor16_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// reductions over the 4 lanes (g = 0..3) that share a query column
__device__ __forceinline__ float col_max(float x) { return xor32_max(xor16_max(x)); }
__device__ __forceinline__ float col_add(float x) { return xor32_add(xor16_add(x)); }

// 4 consecutive entries of a bias / mask row as floats; columns >= n read as `pad`.
template <bool VEC, class T>
__device__ __forceinline__ void load_side4(const T* row, int c0, int n, float pad, float* x) {
    typedef T TV4 __attribute__((ext_vector_type(4)));
    if (VEC) {   // n % 8 == 0 and rows 16-byte aligned: a group of 4 is all real or all padding
        if (c0 < n) {
            const TV4 v = *reinterpret_cast<const TV4*>(row + c0);
#pragma unroll
            for (int i = 0; i < 4; i++) x[i] = (float)v[i];
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) x[i] = pad;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = (c0 + i < n) ? (float)row[c0 + i] : pad;
    }
}

// NT = compile-time bound on the 16-key tiles of a unit (N <= 16 NT); the workgroup has
// ceil(N / 16) wavefronts.
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC>
__global__ void __launch_bounds__(64 * NT) fwd_resident_kernel(const FwdParams p) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    constexpr int ROWS = 16 * NT;
    constexpr int S = kLdsStride;

    __shared__ __attribute__((aligned(16))) SE lds_K[2][ROWS * S];
    __shared__ __attribute__((aligned(16))) E lds_V[2][ROWS * S];

    const int N = p.n;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l16 = lane & 15;       // query column inside the wavefront's 16 rows
    const int g = lane >> 4;         // accumulator rows 4g .. 4g+3, operand k-slots 8g .. 8g+7

    const int h = blockIdx.x / p.groups;
    const int grp = blockIdx.x - h * p.groups;

    float scale2;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        scale2 = expf(fminf(ls, kLn100)) * kLog2e;
    } else {
        scale2 = p.default_scale * kLog2e;
    }

    // rows of the staging buffers that no unit ever writes must read as zeros
    for (int i = tid; i < 2 * ROWS * S / 8; i += nthreads) {
        st8<SV8>(&lds_K[0][0] + i * 8, zero8<SV8>());
        st8<V8>(&lds_V[0][0] + i * 8, zero8<V8>());
    }

    const int qi = wave * 16 + l16;
    const bool qv = qi < N;
    const int qc = min(qi, N - 1);

    // ---- resident bias: acc0[kt][i] <-> key 16 kt + 4 g + i of query qi, log2 domain ----
    f32x4 acc0[NT];
    float mb = 0.f, mn = 0.f;
    if (HAS_BIAS) {
        const E* brow = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qc * p.bias_sn;
        mb = -INFINITY;
        mn = INFINITY;
#pragma unroll
        for (int kt = 0; kt < NT; kt++) {
            float x[4];
            load_side4<VEC, E>(brow, 16 * kt + 4 * g, N, -INFINITY, x);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float v = x[i] * kLog2e;      // -inf stays -inf
                acc0[kt][i] = v;
                mb = fmaxf(mb, v);
                mn = fminf(mn, (16 * kt + 4 * g + i < N) ? v : INFINITY);
            }
        }
        mb = col_max(mb);
        mn = -col_max(-mn);
        if (!(mb > -INFINITY)) { mb = 0.f; mn = 0.f; }   // a row of -inf bias: nothing to bound
    } else {
#pragma unroll
        for (int kt = 0; kt < NT; kt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc0[kt][i] = (16 * kt + 4 * g + i < N) ? 0.f : -INFINITY;
    }
    const float m_fixed = mb + scale2;     // upper bound of every logit of this row (mask <= 0)
#pragma unroll
    for (int kt = 0; kt < NT; kt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc0[kt][i] -= m_fixed;
    // the wavefront takes the maximum-free path if the bound is tight enough for all its rows
    float range = (mb - mn == mb - mn) ? mb - mn : INFINITY;   // NaN / inf ranges disable it
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) range = fmaxf(range, __shfl_xor(range, off));
    const bool wave_fast = (DT == FWA2_BF16) && (2.f * scale2 + range <= kGapLimit);

    // ---- per-unit fetch (into registers) and staging (registers -> LDS) ----
    const int srow = tid >> 2;             // staged row of this thread (< 16 * waves <= ROWS)
    const int sc8 = (tid & 3) * 8;
    auto fetch = [&](int b, V8& kk, V8& vv, V8& qq) __attribute__((always_inline)) {
        kk = zero8<V8>(); vv = zero8<V8>(); qq = zero8<V8>();
        if (srow < N) {
            kk = ld8<V8>(reinterpret_cast<const E*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + (int64_t)srow * p.k.sn + sc8);
            vv = ld8<V8>(reinterpret_cast<const E*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + (int64_t)srow * p.v.sn + sc8);
        }
        if (qv) qq = ld8<V8>(reinterpret_cast<const E*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)qi * p.q.sn + 8 * g);
    };
    auto stage = [&](int buf, V8 kk, V8 vv) __attribute__((always_inline)) {
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
        st8<SV8>(&lds_K[buf][srow * S + sc8], kn);
        st8<V8>(&lds_V[buf][srow * S + sc8], vv);
    };

    int b = grp;
    V8 kk, vv, qq;
    __syncthreads();                       // zero fill done
    if (b < p.bw) {
        fetch(b, kk, vv, qq);
        stage(0, kk, vv);
    }
    __syncthreads();
    int cur = 0;

    while (b < p.bw) {
        const int bn = b + p.groups;
        // ---- Q operand: normalise, fold s log2e, round to fp16 ----
        SV8 bq;
        {
            float x[8];
            unpack8(qq, x);
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) ss += x[j] * x[j];
            ss = col_add(ss);
            const float sc = scale2 * inv_norm(ss);
#pragma unroll
            for (int j = 0; j < 8; j++) bq[j] = (SE)(x[j] * sc);
        }
        if (bn < p.bw) fetch(bn, kk, vv, qq);      // in flight while this unit is computed

        const ME* mrow = nullptr;
        bool masked = false, safe = false;
        if (MASK_DT >= 0) {
            const int w = b % p.n_windows;
            const int fl = p.mask_live ? p.mask_live[w] : 1;
            masked = fl != 0;
            safe = (fl & 2) != 0;
            mrow = reinterpret_cast<const ME*>(p.mask) + w * p.mask_sw + (int64_t)qc * p.mask_sn;
        }

        const SE* Kb = &lds_K[cur][0];
        const E* Vb = &lds_V[cur][0];
        f32x4 oacc[2];
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int i = 0; i < 4; i++) oacc[dt][i] = 0.f;
        float l_run = 0.f;     // online path: this lane's share of the running row sum
        float m_run = 0.f;     // online path: running maximum relative to m_fixed
        bool fast_unit = false;

        // scores of keys 32 kp .. 32 kp + 31 (tile A: rows 4g+i, tile B: rows 16+4g+i)
        auto scores = [&](int kp, bool with_mask, f32x4& s0, f32x4& s1) __attribute__((always_inline)) {
            const SV8 a0 = ld8<SV8>(Kb + (32 * kp + l16) * S + 8 * g);
            const SV8 a1 = ld8<SV8>(Kb + (32 * kp + 16 + l16) * S + 8 * g);
            s0 = Elem<kScoreDT>::mfma16(a0, bq, acc0[2 * kp]);
            s1 = Elem<kScoreDT>::mfma16(a1, bq, acc0[2 * kp + 1]);
            if (MASK_DT >= 0 && with_mask) {
                float x0[4], x1[4];
                load_side4<VEC, ME>(mrow, 32 * kp + 4 * g, N, 0.f, x0);
                load_side4<VEC, ME>(mrow, 32 * kp + 16 + 4 * g, N, 0.f, x1);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    s0[i] = fmaf(x0[i], kLog2e, s0[i]);
                    s1[i] = fmaf(x1[i], kLog2e, s1[i]);
                }
            }
        };
        // FAST: the row sum comes out of a third MFMA against a tile of ones, i.e. it sums the
        // ROUNDED P~ values that also enter the product with V: o is then an exact convex
        // combination of V rows, and the sum costs no VALU work.
        f32x4 lacc;
#pragma unroll
        for (int i = 0; i < 4; i++) lacc[i] = 0.f;
        V8 ones;
#pragma unroll
        for (int j = 0; j < 8; j++) ones[j] = (E)1.0f;
        auto pv = [&](int kp, const f32x4& s0, const f32x4& s1, bool sum_by_mfma) __attribute__((always_inline)) {
            V8 bp;
#pragma unroll
            for (int i = 0; i < 4; i++) { bp[i] = (E)s0[i]; bp[4 + i] = (E)s1[i]; }
            if (sum_by_mfma) lacc = Elem<DT>::mfma16(ones, bp, lacc);
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                const E* vlo = Vb + (32 * kp + 4 * g + (l16 >> 2)) * S + 16 * dt + 4 * (l16 & 3);
                const V8 av = lds_tr8<DT>(vlo, vlo + 16 * S);
                oacc[dt] = Elem<DT>::mfma16(av, bp, oacc[dt]);
            }
        };

        if (wave_fast && (!masked || safe)) {
            fast_unit = true;
            auto body = [&](bool with_mask) __attribute__((always_inline)) {
#pragma unroll
                for (int kp = 0; kp < NT / 2; kp++) {
                    if (32 * kp < N) {
                        f32x4 s0, s1;
                        scores(kp, with_mask, s0, s1);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            s0[i] = fast_exp2(s0[i]);
                            s1[i] = fast_exp2(s1[i]);
                        }
                        pv(kp, s0, s1, true);
                    }
                }
            };
            if (masked) body(true); else body(false);
        } else {
            m_run = -INFINITY;
#pragma unroll
            for (int kp = 0; kp < NT / 2; kp++) {
                if (32 * kp < N) {
                    f32x4 s0, s1;
                    scores(kp, masked, s0, s1);
                    float bm = fmaxf(fmaxf(s0[0], s0[1]), fmaxf(s0[2], s0[3]));
                    bm = fmaxf(bm, fmaxf(fmaxf(s1[0], s1[1]), fmaxf(s1[2], s1[3])));
                    bm = col_max(bm);
                    const float m_new = fmaxf(m_run, bm);
                    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                    const float alpha = fast_exp2(m_run - m_use);
                    m_run = m_new;
                    float ps = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        s0[i] = fast_exp2(s0[i] - m_use);
                        s1[i] = fast_exp2(s1[i] - m_use);
                        ps += s0[i] + s1[i];
                    }
                    l_run = l_run * alpha + ps;
#pragma unroll
                    for (int dt = 0; dt < 2; dt++)
#pragma unroll
                        for (int i = 0; i < 4; i++) oacc[dt][i] *= alpha;
                    pv(kp, s0, s1, false);
                }
            }
        }

        // ---- normalise, write o (input dtype) and lse (natural log, fp32) ----
        const float l_tot = fast_unit ? lacc[0] : col_add(l_run);
        const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        if (qv) {
            E* orow = reinterpret_cast<E*>(const_cast<void*>(p.o.ptr)) + b * p.o.sb + h * p.o.sh + (int64_t)qi * p.o.sn;
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                V4 ov;
#pragma unroll
                for (int i = 0; i < 4; i++) ov[i] = (E)(oacc[dt][i] * inv_l);
                *reinterpret_cast<V4*>(orow + 16 * dt + 4 * g) = ov;
            }
            if (g == 0) {
                const float lse = l_tot > 0.f ? (m_fixed + m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
                p.lse[b * p.lse_sb + h * p.lse_sh + qi] = lse;
            }
        }

        if (bn < p.bw) stage(cur ^ 1, kk, vv);
        __syncthreads();       // next unit staged; everybody is done with the current buffers
        cur ^= 1;
        b = bn;
    }
}

// ---- host side -----------------------------------------------------------------
int forward_resident_supported(int n) { return n >= 1 && n <= 256; }

template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC>
static hipError_t launch_nt(FwdParams p, hipStream_t st) {
    const int waves = (p.n + 15) / 16;
    static const int fit = [&] {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC>,
                                                         64 * NT, 0) != hipSuccess || n < 1)
            n = 1;
        return n;
    }();
    // the runtime's figure is for full 64 NT-thread groups; smaller groups only fit better
    int groups = (p.cus * fit) / p.heads;
    if (groups < 1) groups = 1;
    if (groups > p.bw) groups = p.bw;
    p.groups = groups;
    hipLaunchKernelGGL((fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC>), dim3(p.heads * groups), dim3(64 * waves), 0, st, p);
    return hipGetLastError();
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_mask(const FwdParams& p, hipStream_t st) {
    const int nt = p.n <= 64 ? 4 : (p.n <= 128 ? 8 : 16);
    if (p.side_vec) {
        if (nt == 4) return launch_nt<DT, HAS_BIAS, MASK_DT, 4, true>(p, st);
        if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, true>(p, st);
        return launch_nt<DT, HAS_BIAS, MASK_DT, 16, true>(p, st);
    }
    if (nt == 4) return launch_nt<DT, HAS_BIAS, MASK_DT, 4, false>(p, st);
    if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, false>(p, st);
    return launch_nt<DT, HAS_BIAS, MASK_DT, 16, false>(p, st);
}

template <int DT>
static hipError_t launch_dt(const FwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    if (has_bias) {
        if (mask_dt < 0) return launch_mask<DT, true, -1>(p, st);
        if (mask_dt == FWA2_F32) return launch_mask<DT, true, FWA2_F32>(p, st);
        return launch_mask<DT, true, DT>(p, st);
    }
    if (mask_dt < 0) return launch_mask<DT, false, -1>(p, st);
    if (mask_dt == FWA2_F32) return launch_mask<DT, false, FWA2_F32>(p, st);
    return launch_mask<DT, false, DT>(p, st);
}

hipError_t launch_forward_resident(const FwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, st);
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st);
}

}  // namespace fwa2
