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
// Per unit: K and V rows of the NEXT unit are fetched straight into an LDS
// landing area (global_load_lds, no registers held) before the tiles of the
// current one are computed; afterwards every wavefront normalises the 16 rows
// it fetched into the other half of a double buffer; one barrier per unit.
// Units whose window mask is live go through a second launch of the MASKED
// instantiation, so the common unmasked code carries no mask registers.
#include "fwa2_common.hpp"

namespace fwa2 {

// NT = compile-time bound on the 16-key tiles of a unit (N <= 16 NT); the workgroup has
// ceil(N / 16) wavefronts.
// MASKED: this launch handles the units whose window mask is live; the other units (or all, when
// there is no mask) go through the MASKED = false instantiation.
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MASKED>
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
    __shared__ __attribute__((aligned(16))) E lds_rawK[ROWS * 32];   // landing area: unpadded 64-byte rows
    __shared__ __attribute__((aligned(16))) E lds_rawV[ROWS * 32];
    __shared__ uint8_t lds_live[kLiveCache];       // copy of the per-window mask flags
    __shared__ uint16_t lds_list[kLiveCache];      // windows of this launch's class, ascending
    __shared__ int lds_count;

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
    for (int i = tid; i < ROWS * 32 / 8; i += nthreads) {
        st8<V8>(lds_rawK + i * 8, zero8<V8>());
        st8<V8>(lds_rawV + i * 8, zero8<V8>());
    }

    const int qi = wave * 16 + l16;
    const bool qv = qi < N;
    const int qc = min(qi, N - 1);

    // ---- resident bias, log2 domain.  Keys are taken 32 at a time; of such a group this lane holds
    // keys 8g .. 8g+7: acc0[2kp][i] <-> key 32kp + 8g + i, acc0[2kp+1][i] <-> key 32kp + 8g + 4 + i
    // (so bias and mask rows are read 8 consecutive entries at a time) ----
    f32x4 acc0[NT];
    float mb = 0.f, mn = 0.f;
    if (HAS_BIAS) {
        const E* brow = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qc * p.bias_sn;
        mb = -INFINITY;
        mn = INFINITY;
#pragma unroll
        for (int kp = 0; kp < NT / 2; kp++) {
            const auto raw = load_raw8<VEC, E>(brow, 32 * kp + 8 * g, N, -INFINITY);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float v = (float)raw[j] * kLog2e;      // -inf stays -inf
                acc0[2 * kp + (j >> 2)][j & 3] = v;
                mb = fmaxf(mb, v);
                mn = fminf(mn, (32 * kp + 8 * g + j < N) ? v : INFINITY);
            }
        }
        mb = col_max(mb);
        mn = -col_max(-mn);
        if (!(mb > -INFINITY)) { mb = 0.f; mn = 0.f; }   // a row of -inf bias: nothing to bound
    } else {
#pragma unroll
        for (int kt = 0; kt < NT; kt++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                acc0[kt][i] = (32 * (kt >> 1) + 8 * g + 4 * (kt & 1) + i < N) ? 0.f : -INFINITY;
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

    // ---- which units belong to this launch.  With cached flags the windows of this launch's class
    // (mask live or not) are listed once, and the units are dealt out by their rank within the
    // class, so every workgroup of the head gets the same number of them whatever the pattern of
    // masked windows. ----
    const bool listed = MASK_DT >= 0 && p.mask_live && p.n_windows <= kLiveCache;
    if (listed) {
        for (int i = tid; i < p.n_windows; i += nthreads) lds_live[i] = p.mask_live[i];
        __syncthreads();
        if (wave == 0) {
            int cnt = 0;
            for (int base = 0; base < p.n_windows; base += 64) {
                const int w = base + lane;
                const bool in = w < p.n_windows && ((lds_live[w] != 0) == MASKED);
                const unsigned long long bal = __ballot(in);
                if (in) lds_list[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = (uint16_t)w;
                cnt += __popcll(bal);
            }
            if (lane == 0) lds_count = cnt;
        }
        __syncthreads();
    }
    const int cnt = listed ? lds_count : 0;
    const int total = listed ? ((p.bw + p.n_windows - 1) / p.n_windows) * cnt : p.bw;   // ranks to deal out
    auto unit_of = [&](int t) -> int {
        if (!listed) return t;
        const int img = t / cnt;
        // the same for every lane: keep it (and the addresses derived from it) in scalar registers
        return __builtin_amdgcn_readfirstlane(img * p.n_windows + (int)lds_list[t - img * cnt]);
    };
    auto flags_of = [&](int b) -> int {
        const int w = b % p.n_windows;
        return __builtin_amdgcn_readfirstlane(listed ? (int)lds_live[w] : (int)p.mask_live[w]);
    };
    // first rank >= t (in steps of the group count) that names an existing unit of this launch
    auto rank_from = [&](int t) -> int {
        for (; t < total; t += p.groups) {
            const int b = unit_of(t);
            if (b >= p.bw) continue;
            if (listed || MASK_DT < 0 || !p.mask_live || ((flags_of(b) != 0) == MASKED)) return t;
        }
        return total;
    };
    // ---- per-unit fetch: every wavefront brings in the 16 K and V rows it will stage (lane i lands
    // at 16 i bytes from the wavefront's base) and its own 16 query rows ----
    const int frow = wave * 16 + (lane >> 2);      // K / V row of this lane
    const int fc8 = (lane & 3) * 8;
    auto fetch = [&](int b, V8& qq) __attribute__((always_inline)) {
        if (frow < N) {
            const E* kp = reinterpret_cast<const E*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + (int64_t)frow * p.k.sn + fc8;
            const E* vp = reinterpret_cast<const E*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + (int64_t)frow * p.v.sn + fc8;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kp,
                                             (__attribute__((address_space(3))) void*)(lds_rawK + wave * 16 * 32), 16, 0, kStreamPolicy);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vp,
                                             (__attribute__((address_space(3))) void*)(lds_rawV + wave * 16 * 32), 16, 0, kStreamPolicy);
        }
        qq = zero8<V8>();
        if (qv) qq = ld8<V8>(reinterpret_cast<const E*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)qi * p.q.sn + 8 * g);
    };
    // landing area -> tiles: K normalised and rounded to fp16, V as is (rows >= n stay zero)
    auto stage = [&](int buf) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // this wavefront's rows have landed
        const V8 kk = ld8<V8>(lds_rawK + frow * 32 + fc8);
        const V8 vv = ld8<V8>(lds_rawV + frow * 32 + fc8);
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
        st8<SV8>(&lds_K[buf][frow * S + fc8], kn);
        st8<V8>(&lds_V[buf][frow * S + fc8], vv);
    };

    __syncthreads();                       // zero fill done
    int t = rank_from(grp);
    V8 qq = zero8<V8>();
    if (t < total) {
        fetch(unit_of(t), qq);
        stage(0);
    }
    __syncthreads();
    int cur = 0;

    while (t < total) {
        const int b = unit_of(t);
        const int tn = rank_from(t + p.groups);
        const int bn = tn < total ? unit_of(tn) : p.bw;
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
        if (bn < p.bw) fetch(bn, qq);      // in flight while this unit is computed

        const ME* mrow = nullptr;
        constexpr bool masked = MASKED;
        bool safe = false;
        if (MASKED) {
            const int w = b % p.n_windows;
            safe = p.mask_live ? (flags_of(b) & 2) != 0 : false;
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

        typedef ME MV8 __attribute__((ext_vector_type(8)));
        // scores of keys 32 kp .. 32 kp + 31: MFMA tile A holds keys 8r/4 + r%4 in its rows r, tile B
        // the keys 4 further on, so that this lane's 8 values are keys 8g .. 8g+7 of the group
        auto scores = [&](int kp, bool with_mask, const MV8& mk, f32x4& s0, f32x4& s1) __attribute__((always_inline)) {
            const int krow = 32 * kp + 8 * (l16 >> 2) + (l16 & 3);
            const SV8 a0 = ld8<SV8>(Kb + krow * S + 8 * g);
            const SV8 a1 = ld8<SV8>(Kb + (krow + 4) * S + 8 * g);
            s0 = Elem<kScoreDT>::mfma16(a0, bq, acc0[2 * kp]);
            s1 = Elem<kScoreDT>::mfma16(a1, bq, acc0[2 * kp + 1]);
            if (MASK_DT >= 0 && with_mask) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    s0[i] = fmaf((float)mk[i], kLog2e, s0[i]);
                    s1[i] = fmaf((float)mk[4 + i], kLog2e, s1[i]);
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
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4: this lane's accumulators hold d = 8g + 4dt + i
                const E* vlo = Vb + (32 * kp + 8 * g + (l16 >> 2)) * S + 8 * (l16 & 3) + 4 * dt;
                const V8 av = lds_tr8<DT>(vlo, vlo + 4 * S);
                oacc[dt] = Elem<DT>::mfma16(av, bp, oacc[dt]);
            }
        };

        if (wave_fast && (!masked || safe)) {
            fast_unit = true;
            auto body = [&](bool with_mask) __attribute__((always_inline)) {
                // mask rows travel two key groups ahead of their use
                MV8 mq[2];
                if (MASK_DT >= 0 && with_mask) {
                    mq[0] = load_raw8<VEC, ME>(mrow, 8 * g, N, 0.f);
                    mq[1] = load_raw8<VEC, ME>(mrow, 32 + 8 * g, N, 0.f);
                }
#pragma unroll
                for (int kp = 0; kp < NT / 2; kp++) {
                    if (32 * kp < N) {
                        f32x4 s0, s1;
                        scores(kp, with_mask, mq[kp & 1], s0, s1);
                        if (MASK_DT >= 0 && with_mask && kp + 2 < NT / 2)
                            mq[kp & 1] = load_raw8<VEC, ME>(mrow, 32 * (kp + 2) + 8 * g, N, 0.f);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            s0[i] = fast_exp2(s0[i]);
                            s1[i] = fast_exp2(s1[i]);
                        }
                        pv(kp, s0, s1, true);
                    }
                }
            };
            body(MASKED);
        } else {
            m_run = -INFINITY;
#pragma unroll
            for (int kp = 0; kp < NT / 2; kp++) {
                if (32 * kp < N) {
                    f32x4 s0, s1;
                    MV8 mk;
                    if (MASK_DT >= 0 && masked) mk = load_raw8<VEC, ME>(mrow, 32 * kp + 8 * g, N, 0.f);
                    scores(kp, masked, mk, s0, s1);
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

        if (bn < p.bw) stage(cur ^ 1);     // before the stores below, so the wait covers only the fetch
        // ---- normalise, write o (input dtype) and lse (natural log, fp32) ----
        const float l_tot = fast_unit ? lacc[0] : col_add(l_run);
        const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        if (qv) {
            E* orow = reinterpret_cast<E*>(const_cast<void*>(p.o.ptr)) + b * p.o.sb + h * p.o.sh + (int64_t)qi * p.o.sn;
            V8 ov;
#pragma unroll
            for (int j = 0; j < 8; j++) ov[j] = (E)(oacc[j >> 2][j & 3] * inv_l);
            st8_stream<V8>(orow + 8 * g, ov);
            if (g == 0) {
                const float lse = l_tot > 0.f ? (m_fixed + m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
                p.lse[b * p.lse_sb + h * p.lse_sh + qi] = lse;
            }
        }

        __syncthreads();       // next unit staged; everybody is done with the current buffers
        cur ^= 1;
        t = tn;
    }
}

// ---- host side -----------------------------------------------------------------
int forward_resident_supported(int n) { return n >= 1 && n <= 256; }

template <class K>
static int resident_fit(K kern, int threads) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, threads, 0) != hipSuccess || n < 1) n = 1;
    return n;
}

template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC>
static hipError_t launch_nt(FwdParams p, hipStream_t st) {
    const int waves = (p.n + 15) / 16;
    // the runtime's figure is for full 64 NT-thread groups; smaller groups only fit better
    static const int fit_plain = resident_fit(fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, false>, 64 * NT);
    static const int fit_masked = MASK_DT >= 0 ? resident_fit(fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, true>, 64 * NT) : 1;
    auto groups_for = [&](int fit) {
        int groups = (p.cus * fit) / p.heads;
        if (groups < 1) groups = 1;
        if (groups > p.bw) groups = p.bw;
        return groups;
    };
    // units with an all-zero mask (or every unit when there is no mask) ...
    if (MASK_DT < 0 || p.mask_live != nullptr) {
        p.groups = groups_for(fit_plain);
        hipLaunchKernelGGL((fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, false>), dim3(p.heads * p.groups),
                           dim3(64 * waves), 0, st, p);
    }
    // ... and the units whose mask is live
    if (MASK_DT >= 0) {
        p.groups = groups_for(fit_masked);
        hipLaunchKernelGGL((fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, true>), dim3(p.heads * p.groups),
                           dim3(64 * waves), 0, st, p);
    }
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
