// Backward for windows of up to 64 tokens in ONE pass over q, k, v, o, dO: dq, dk, dv,
// dbias and dlogit_scale from the same persistent workgroups.
//
// Replaces _bwd_preprocess_do_o_dot and _bwd_kernel
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:6-51, 84-564) for N <= 64.  Longer
// windows use the key-side kernel (fwa2_bwd.hip) plus the query-side kernel
// (fwa2_bwd_dq_resident.hip), which read q, k, v, dO twice; at these sizes the operator is
// bound by HBM traffic, and a whole window's P and dZ (2 x 64 x 64 values) fit in LDS.
//
// Skeleton of the resident query-side kernel: a workgroup belongs to one head, every
// wavefront owns 16 query rows and holds (bias [+ mask]) * log2e - m for them in the register
// layout of the score accumulators.  The rows of the next unit travel in registers while the
// current unit is computed (21 registers per lane; no landing area, so three workgroups fit a CU).
// Per unit:
//   phase A (wavefront = 16 queries, lane = query, registers = keys)
//     S^T - m = K_hat Q_hat^T,  dP^T - delta = V dO^T,  e = 2^(S^T - lse2),  dZ^T = e (dP^T - delta)
//     dQ_hat^T += K_hat^T dZ^T;  dbias tile += dZ (registers, for the whole launch)
//     e and dZ go to two [query][key] tiles in LDS
//   barrier
//   phase B (wavefront = 16 keys): the tiles come back through transposing LDS reads as MFMA
//     operands whose contraction index is the query, so every wavefront sums over all queries
//     itself:  dV^T = dO^T P,  dK_hat^T = Q_hat^T dZ  -- no partial sums between wavefronts.
// delta = rowsum(o * dO) is computed on the spot from the landed rows.
#include "fwa2_common.hpp"

namespace fwa2 {

// The walk of one workgroup (head h, workgroup grp of the `groups` its class of windows has for that head) over its
// units; its dbias tile and dscale partial go to slot `slot` of the head.
// MASKED: the class of windows whose mask is live (the resident tile then holds bias + the window's mask).
// MAPPED: rows are addressed through the window map (cyclic shift + window partition done here).
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MASKED, bool MAPPED>
__device__ __forceinline__ void bwd_fused_body(const BwdParams& p, const int h, const int grp, const int groups, const int slot) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    typedef typename Elem<kScoreDT>::V4 SV4;
    constexpr int ROWS = 16 * NT;
    constexpr int S = kLdsStride;         // row stride of the 32-column tiles
    constexpr int PS = ROWS + 8;          // row stride of the [query][key] tiles

    // (arrays shared by the two bodies a kernel may run, one per class of windows)
    SE* lds_K = shared_array<SE, ROWS * S, 0>();           // k_hat of the current unit
    E* lds_V = shared_array<E, ROWS * S, 1>();
    float* lds_kinv = shared_array<float, ROWS, 2>();      // 1 / max(|k|, eps), negated when |k| <= eps
    SE* lds_Qs = shared_array<SE, ROWS * S, 3>();          // q_hat s log2e of the current unit
    E* lds_dOs = shared_array<E, ROWS * S, 4>();           // dO (times w when folded) of the current unit
    E* lds_Pt = shared_array<E, ROWS * PS, 5>();           // e,  [query][key]
    SE* lds_Zt = shared_array<SE, ROWS * PS, 6>();         // dZ, [query][key]
    uint8_t* lds_live = shared_array<uint8_t, kLiveCache, 7>();
    uint16_t* lds_list = shared_array<uint16_t, kLiveCache, 8>();
    int& lds_count = *shared_array<int, 4, 9>();
    float* lds_red = shared_array<float, NT, 10>();

    const int N = p.n;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l16 = lane & 15;
    const int g = lane >> 4;

    float s_true;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        s_true = expf(fminf(ls, kLn100));
    } else {
        s_true = p.default_scale;
    }
    const float scale2 = s_true * kLog2e;

    // every tile row is rewritten for every unit (rows >= n with zeros), nothing to clear up front

    const int qrow = wave * 16 + l16;       // this lane's query in phase A

    // ---- resident tile (as in fwa2_fwd_resident.hip): acc0[2kp][i] <-> key 32kp + 8g + i,
    // acc0[2kp+1][i] <-> key 32kp + 8g + 4 + i; (bias + mask) * log2e minus the row bound
    // m_fixed = s log2e + max_j (bias2 + mask2)[j] ----
    f32x4 acc0[NT];
    float m_fixed = 0.f;
    auto build_tile = [&](int w) __attribute__((always_inline)) {
        int ln = lane;                     // re-derived per call, so that no row address lives across units
        if (MASKED) asm volatile("" : "+v"(ln));
        const int g = ln >> 4;
        const int qr = min(wave * 16 + (ln & 15), N - 1);
        const E* brow = nullptr;
        const ME* mrow = nullptr;
        if (HAS_BIAS) brow = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qr * p.bias_sn;
        if (MASKED) mrow = reinterpret_cast<const ME*>(p.mask) + w * p.mask_sw + (int64_t)qr * p.mask_sn;
        float mb = -INFINITY;
#pragma unroll
        for (int kp = 0; kp < NT / 2; kp++) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = (32 * kp + 8 * g + j < N) ? 0.f : -INFINITY;
            if (HAS_BIAS) {
                const auto raw = load_raw8<VEC, E>(brow, 32 * kp + 8 * g, N, 0.f);
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] += (float)raw[j] * kLog2e;
            }
            if (MASKED) {
                const auto raw = load_raw8<VEC, ME>(mrow, 32 * kp + 8 * g, N, 0.f);
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = fmaf((float)raw[j], kLog2e, v[j]);
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc0[2 * kp + (j >> 2)][j & 3] = v[j];
                mb = fmaxf(mb, v[j]);
            }
        }
        mb = col_max(mb);
        if (!(mb > -INFINITY)) mb = 0.f;        // every key of the row removed: nothing to bound
        m_fixed = mb + scale2;
#pragma unroll
        for (int kt = 0; kt < NT; kt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc0[kt][i] -= m_fixed;
    };
    // w = 2^(m - lse2) lies in [1/N, 2^(2 s log2e)]: it may be folded into dO when that cannot leave
    // the bf16 range
    const bool fold = (DT == FWA2_BF16) && (2.f * scale2 <= kGapLimit);

    // ---- which units belong to this class of windows (same dealing as in fwa2_fwd_resident.hip) ----
    const int nw = MASK_DT >= 0 ? p.n_windows : 1;
    const bool listed = MASK_DT >= 0 && p.mask_live != nullptr;
    if (listed) {
        for (int i = tid; i < nw; i += nthreads) lds_live[i] = p.mask_live[i];
        __syncthreads();
        if (wave == 0) {
            int c = 0;
            for (int base = 0; base < nw; base += 64) {
                const int w = base + lane;
                const bool in = w < nw && ((lds_live[w] != 0) == MASKED);
                const unsigned long long bal = __ballot(in);
                if (in) lds_list[c + __popcll(bal & ((1ull << lane) - 1ull))] = (uint16_t)w;
                c += __popcll(bal);
            }
            if (lane == 0) lds_count = c;
        }
        __syncthreads();
    }
    const int cnt = listed ? __builtin_amdgcn_readfirstlane(lds_count) : nw;    // windows of this class
    const int n_img = p.bw / nw;
    auto window_at = [&](int wi) -> int {
        return listed ? __builtin_amdgcn_readfirstlane((int)lds_list[wi]) : wi;
    };
    // MASKED: the units in window-major order, t = wi * n_img + img, are cut into one stretch per workgroup (lengths
    // differ by at most one), so a workgroup changes its window once or twice at most
    const int64_t units_m = (int64_t)cnt * n_img;
    const int t_first = MASKED ? (int)(units_m * grp / groups) : 0;
    const int t_count = MASKED ? (int)(units_m * (grp + 1) / groups) - t_first : 0;
    struct Cursor { int wi, img, left; };
    auto valid = [&](const Cursor& c) -> bool { return MASKED ? c.left > 0 : c.img < n_img; };
    auto first = [&]() -> Cursor {
        Cursor c;
        c.left = t_count;
        if (MASKED) { c.wi = t_first / n_img; c.img = t_first - c.wi * n_img; }
        else { c.img = cnt > 0 ? grp / cnt : n_img; c.wi = cnt > 0 ? grp - c.img * cnt : 0; }
        return c;
    };
    auto next = [&](Cursor c) -> Cursor {
        if (MASKED) {
            c.left -= 1;
            c.img += 1;
            if (c.img >= n_img) { c.img = 0; c.wi += 1; }
        } else {
            const int t = c.img * cnt + c.wi + groups;
            c.img = t / cnt;
            c.wi = t - c.img * cnt;
        }
        return c;
    };
    auto unit_of = [&](const Cursor& c) -> int { return c.img * nw + window_at(c.wi); };

    // ---- per-unit fetch, one unit ahead, into registers: 16 bytes of a k and a v row (the 16 rows
    // this wavefront stages, 4 lanes per row) and 16 bytes of the q, dO and o rows of this lane's
    // query in the operand layout (lane (query, g) takes columns 8g .. 8g+7); rows >= n read as zeros ----
    struct Rows { V8 k, v, q, dO, o; float lse; };
    auto ldrow = [&](const T4& t, int b, int row, int col) -> V8 {
        return ld8<V8>(row_ptr<MAPPED, E>(t, p.map, b, h, row, col));
    };
    auto fetch = [&](int b, Rows& r) __attribute__((always_inline)) {
        int ln = lane;                     // re-derived per call: no address lives across the unit loop
        asm volatile("" : "+v"(ln));
        const int frow = wave * 16 + (ln >> 2), fc8 = (ln & 3) * 8;
        r.k = zero8<V8>(); r.v = zero8<V8>();
        if (frow < N) { r.k = ldrow(p.k, b, frow, fc8); r.v = ldrow(p.v, b, frow, fc8); }
        const int q = wave * 16 + (ln & 15), c8 = (ln >> 4) * 8;
        r.q = zero8<V8>(); r.dO = zero8<V8>(); r.o = zero8<V8>();
        r.lse = -INFINITY;
        if (q < N) {
            r.q = ldrow(p.q, b, q, c8); r.dO = ldrow(p.d_o, b, q, c8); r.o = ldrow(p.o, b, q, c8);
            r.lse = p.lse[b * p.lse_sb + h * p.lse_sh + q];
        }
    };
    // k, v rows -> tiles: K normalised and rounded to fp16, V as is
    auto stage = [&](const Rows& r) __attribute__((always_inline)) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int frow = wave * 16 + (ln >> 2), fc8 = (ln & 3) * 8;
        float x[8];
        unpack8(r.k, x);
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) ss += x[j] * x[j];
        ss = quad_add(ss);
        const float inv = inv_norm(ss);
        SV8 kn;
#pragma unroll
        for (int j = 0; j < 8; j++) kn[j] = (SE)(x[j] * inv);
        st8<SV8>(lds_K + frow * S + fc8, kn);
        st8<V8>(lds_V + frow * S + fc8, r.v);
        if ((ln & 3) == 0) lds_kinv[frow] = (sqrtf(ss) > kNormEps) ? inv : -inv;
    };

    // ---- dbias tile of this wavefront's queries, in the layout of the resident tile ----
    float dbacc[NT / 2][8];
#pragma unroll
    for (int kp = 0; kp < NT / 2; kp++)
#pragma unroll
        for (int j = 0; j < 8; j++) dbacc[kp][j] = 0.f;

    // this lane's key in phase B: the transposing reads hand lane n the column 8 (n / 4) + n % 4 of a
    // 32-column group, wavefront pairs share a group and take its two interleaved halves
    const int kcol0 = 32 * (wave >> 1) + 4 * (wave & 1);

    Cursor c = first();
    int tile_wi = -1;                      // window index the resident tile was built for
    if (!MASKED) build_tile(0);
    Rows nx;
    nx.k = zero8<V8>(); nx.v = zero8<V8>(); nx.q = zero8<V8>(); nx.dO = zero8<V8>(); nx.o = zero8<V8>();
    nx.lse = -INFINITY;
    if (valid(c)) {
        fetch(unit_of(c), nx);
        stage(nx);
    }
    __syncthreads();
    float ds_acc = 0.f;        // sum over this lane's queries of q_hat . dq_hat

    while (valid(c)) {
        const int b = unit_of(c);
        const Cursor cn = next(c);
        const bool more = valid(cn);
        if (MASKED && c.wi != tile_wi) {
            build_tile(window_at(c.wi));
            tile_wi = c.wi;
        }

        // ---- this unit's query-side operands out of the landed rows; delta = rowsum(o * dO) ----
        SV8 bq;
        V8 bd;
        f32x4 ndv, dqacc[2];
        float nl, inv;
        {
            const V8 qcur = nx.q, docur = nx.dO, ocur = nx.o;
            float x[8];
            unpack8(qcur, x);
            float ss = 0.f, dl = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) { ss += x[j] * x[j]; dl += (float)ocur[j] * (float)docur[j]; }
            ss = col_add(ss);
            dl = col_add(dl);
            inv = 1.0f / fmaxf(sqrtf(ss), kNormEps);
            const float sc = scale2 * inv;
#pragma unroll
            for (int j = 0; j < 8; j++) bq[j] = (SE)(x[j] * sc);
            const float lse = nx.lse;
            // fully masked row (lse = -inf): P = 0
            nl = (lse == -INFINITY) ? -INFINITY : m_fixed - lse * kLog2e;
            float nd;
            if (fold) {
                const float w = fast_exp2(nl);
#pragma unroll
                for (int j = 0; j < 8; j++) bd[j] = (E)((float)docur[j] * w);
                nd = -dl * w;
                nl = 0.f;
            } else {
                bd = docur;
                nd = -dl;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) { dqacc[0][i] = 0.f; dqacc[1][i] = 0.f; ndv[i] = nd; }
            // the same two operands as row-major tiles, for phase B
            st8<SV8>(lds_Qs + qrow * S + 8 * g, bq);
            st8<V8>(lds_dOs + qrow * S + 8 * g, bd);
        }
        if (more) fetch(unit_of(cn), nx);      // in flight while this unit is computed

        const SE* Kb = lds_K;
        const E* Vb = lds_V;

        // ---- phase A ----
        auto group = [&](int kp, bool folded) __attribute__((always_inline)) {
            const int krow = 32 * kp + 8 * (l16 >> 2) + (l16 & 3);
            SV8 bz;
            V8 pe;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const SV8 ak = ld8<SV8>(Kb + (krow + 4 * half) * S + 8 * g);
                const V8 av = ld8<V8>(Vb + (krow + 4 * half) * S + 8 * g);
                const f32x4 s = Elem<kScoreDT>::mfma16(ak, bq, acc0[2 * kp + half]);
                const f32x4 dp = Elem<DT>::mfma16(av, bd, ndv);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = folded ? fast_exp2(s[i]) : fast_exp2(s[i] + nl);
                    const float dz = e * dp[i];
                    if (HAS_BIAS) dbacc[kp][4 * half + i] += dz;
                    pe[4 * half + i] = (E)e;
                    bz[4 * half + i] = (SE)dz;
                }
            }
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4, so that this lane's accumulators hold d = 8g + 4dt + i
                const SE* klo = Kb + (32 * kp + 8 * g + (l16 >> 2)) * S + 8 * (l16 & 3) + 4 * dt;
                const SV8 akt = lds_tr8<kScoreDT>(klo, klo + 4 * S);
                dqacc[dt] = Elem<kScoreDT>::mfma16(akt, bz, dqacc[dt]);
            }
            // this lane's 8 keys of its query row, for phase B
            st8<V8>(lds_Pt + qrow * PS + 32 * kp + 8 * g, pe);
            st8<SV8>(lds_Zt + qrow * PS + 32 * kp + 8 * g, bz);
        };
        auto body = [&](bool folded) __attribute__((always_inline)) {
#pragma unroll
            for (int kp = 0; kp < NT / 2; kp++)
                if (32 * kp < N) group(kp, folded);
        };
        if (fold) body(true); else body(false);

        // ---- dq: back through q / max(|q|, eps); q_hat . dq_hat is this row's share of dlogit_scale ----
        {
            const float unscale = 1.0f / scale2;
            int ln2 = lane;
            asm volatile("" : "+v"(ln2));
            float qh[8];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                qh[j] = (float)bq[j] * unscale;
                dot += dqacc[j >> 2][j & 3] * qh[j];
            }
            dot = col_add(dot);
            const float proj = inv < 0.5f / kNormEps ? dot : 0.f;      // |q| <= eps: no projection
            const float f = s_true * inv;
            const int q = wave * 16 + (ln2 & 15);
            if (q < N) {
                E* dqrow = const_cast<E*>(row_ptr<MAPPED, E>(p.dq, p.map, b, h, q));
                V8 o8;
#pragma unroll
                for (int j = 0; j < 8; j++) o8[j] = (E)(f * (dqacc[j >> 2][j & 3] - qh[j] * proj));
                st8_stream<V8>(dqrow + 8 * (ln2 >> 4), o8);
                if ((ln2 >> 4) == 0) ds_acc += dot;
            }
        }

        // k_hat row and 1/|k| of this lane's phase-B key, taken while the K tile is still this unit's
        int ln3 = lane;
        asm volatile("" : "+v"(ln3));
        const int n16 = ln3 & 15, g3 = ln3 >> 4;
        const int key = kcol0 + 8 * (n16 >> 2) + (n16 & 3);
        const SV8 krow8 = ld8<SV8>(Kb + key * S + 8 * g3);
        const float ki = lds_kinv[key];

        __syncthreads();       // e, dZ, q_hat and dO tiles of every wavefront are complete; K / V tiles are free
        if (more) stage(nx);   // the next unit's k, v rows have had phase A to arrive

        // ---- phase B: this wavefront's 16 keys against all queries ----
        {
            f32x4 dvacc[2], dkacc[2];
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
#pragma unroll
                for (int i = 0; i < 4; i++) { dvacc[dt][i] = 0.f; dkacc[dt][i] = 0.f; }
#pragma unroll
            for (int ks = 0; ks < NT / 2; ks++) {
                if (32 * ks < N) {
                    const int q8 = 32 * ks + 8 * g;          // first of this lane's 8 queries (operand k-slots)
                    const int poff = (q8 + (l16 >> 2)) * PS + kcol0 + 8 * (l16 & 3);
                    const V8 p8 = lds_tr8<DT>(lds_Pt + poff, lds_Pt + poff + 4 * PS);
                    const SV8 z8 = lds_tr8<kScoreDT>(lds_Zt + poff, lds_Zt + poff + 4 * PS);
#pragma unroll
                    for (int dt = 0; dt < 2; dt++) {
                        const int off = (q8 + (l16 >> 2)) * S + 8 * (l16 & 3) + 4 * dt;
                        const V8 a_do = lds_tr8<DT>(lds_dOs + off, lds_dOs + off + 4 * S);
                        dvacc[dt] = Elem<DT>::mfma16(a_do, p8, dvacc[dt]);
                        const SV8 a_q = lds_tr8<kScoreDT>(lds_Qs + off, lds_Qs + off + 4 * S);
                        dkacc[dt] = Elem<kScoreDT>::mfma16(a_q, z8, dkacc[dt]);
                    }
                }
            }
            // epilogue dk, dv: lane (key, g) holds d = 8g + 4dt + i (16 bytes of a row)
            float x[8], a[8];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                x[j] = (float)krow8[j];
                a[j] = dkacc[j >> 2][j & 3] * kLn2;      // undo the log2e folded into q_hat
                dot += a[j] * x[j];
            }
            dot = xor32_add(xor16_add(dot));
            const float kinv = fabsf(ki);
            const float proj = ki > 0.f ? dot : 0.f;
            if (key < N) {
                E* dkp = const_cast<E*>(row_ptr<MAPPED, E>(p.dk, p.map, b, h, key));
                E* dvp = const_cast<E*>(row_ptr<MAPPED, E>(p.dv, p.map, b, h, key));
                V8 o8, v8;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    o8[j] = (E)(kinv * (a[j] - x[j] * proj));
                    v8[j] = (E)dvacc[j >> 2][j & 3];
                }
                st8_stream<V8>(dkp + 8 * g3, o8);
                st8_stream<V8>(dvp + 8 * g3, v8);
            }
        }

        __syncthreads();       // next unit staged; everybody is done with this unit's tiles
        c = cn;
    }

    // ---- flush: dbias partial tile (key-major, as reduce_kernel reads it) and the dscale partial ----
    if (HAS_BIAS) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int q = wave * 16 + (ln & 15), gg = ln >> 4;
        float* dst = p.part_dbias + ((int64_t)h * p.db_parts + slot) * p.npk_tot * p.r_tot;
#pragma unroll
        for (int kp = 0; kp < NT / 2; kp++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int key = 32 * kp + 8 * gg + j;
                if (key < p.npk_tot && q < p.r_tot) dst[(int64_t)key * p.r_tot + q] = dbacc[kp][j];
            }
    }
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float wsum = wave_sum(ds_acc);
        if (lane == 0) lds_red[wave] = wsum;
        __syncthreads();
        if (tid == 0) {
            float tot = 0.f;
            for (int i = 0; i < (nthreads >> 6); i++) tot += lds_red[i];
            p.part_dscale[(int64_t)h * p.ds_parts + slot] = tot * s_true;
        }
    }
}

// One launch for all the units of a call: without a mask every workgroup runs the plain body; with one, the workgroups
// of a head are split between the windows whose mask is all zero and the others in proportion to their numbers (every
// window has the same number of images) and run side by side.  Without mask flags every window counts as masked.
// Every workgroup owns slot grp of its head's partial tiles.  With a single workgroup per head it runs one class
// after the other and writes two slots.
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MAPPED>
__global__ void __launch_bounds__(64 * NT, 3) bwd_fused_kernel(const BwdParams p) {
    const int groups = p.dq_groups;
    const int h = blockIdx.x / groups;
    const int grp = blockIdx.x - h * groups;
#define FWA2_FUSED_BODY(M, G0, GN, SLOT) bwd_fused_body<DT, HAS_BIAS, MASK_DT, NT, VEC, M, MAPPED>(p, h, G0, GN, SLOT)
    if constexpr (MASK_DT < 0) {
        FWA2_FUSED_BODY(false, grp, groups, grp);
    } else {
        if (groups < 2) {
            FWA2_FUSED_BODY(false, 0, 1, 0);
            __syncthreads();
            FWA2_FUSED_BODY(true, 0, 1, 1);
            return;
        }
        const int nw = p.n_windows;
        int n_masked = nw;
        if (p.mask_live != nullptr) {
            const int lane = threadIdx.x & 63;
            n_masked = 0;
            for (int base = 0; base < nw; base += 64) {
                const int w = base + lane;
                const uint8_t f = w < nw ? p.mask_live[w] : (uint8_t)0;
                n_masked += __popcll(__ballot(f != 0));
            }
            n_masked = __builtin_amdgcn_readfirstlane(n_masked);
        }
        if (n_masked == 0) {
            FWA2_FUSED_BODY(false, grp, groups, grp);
        } else if (n_masked == nw) {
            FWA2_FUSED_BODY(true, grp, groups, grp);
        } else {
            int g_masked = (int)(((int64_t)groups * n_masked + nw / 2) / nw);
            g_masked = g_masked < 1 ? 1 : (g_masked > groups - 1 ? groups - 1 : g_masked);
            const int g_plain = groups - g_masked;
            if (grp < g_plain) FWA2_FUSED_BODY(false, grp, g_plain, grp);
            else FWA2_FUSED_BODY(true, grp - g_plain, g_masked, grp);
        }
    }
#undef FWA2_FUSED_BODY
}

// ---- host side -----------------------------------------------------------------
int backward_fused_supported(int n) { return n >= 1 && n <= 64; }

// Launches the kernel; reports how many partial tiles / dscale partials per head it wrote.
template <int DT, bool HAS_BIAS, int MASK_DT, bool VEC, bool MAPPED>
static hipError_t launch_map(BwdParams p, hipStream_t st, int max_groups, int* parts_out) {
    constexpr int NT = 4;
    // wavefront pairs share a 32-key group in phase B, so there is always an even number of them
    const int waves = 2 * ((p.n + 31) / 32);
    static std::atomic<int> fit_by_device[kFitDevices];
    const int fit = resident_per_cu_cached(bwd_fused_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, MAPPED>, 64 * NT, fit_by_device);
    int groups = (p.cus * fit) / p.heads;
    if (groups < 1) groups = 1;
    if (groups > p.bw) groups = p.bw;
    if (groups > max_groups) groups = max_groups;
    p.dq_groups = groups;
    p.ds_parts = p.db_parts = (MASK_DT >= 0 && groups < 2) ? 2 : groups;
    p.ds_slot0 = p.db_slot0 = 0;
    if (p.ev_start) (void)hipEventRecord(p.ev_start, st);
    hipLaunchKernelGGL((bwd_fused_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, MAPPED>), dim3(p.heads * groups), dim3(64 * waves), 0, st, p);
    if (p.ev_stop) (void)hipEventRecord(p.ev_stop, st);
    *parts_out = p.ds_parts;
    return hipGetLastError();
}

template <int DT, bool HAS_BIAS, int MASK_DT, bool VEC>
static hipError_t launch_vec(const BwdParams& p, hipStream_t st, int max_groups, int* parts_out) {
    if (p.map.nw > 0) return launch_map<DT, HAS_BIAS, MASK_DT, VEC, true>(p, st, max_groups, parts_out);
    return launch_map<DT, HAS_BIAS, MASK_DT, VEC, false>(p, st, max_groups, parts_out);
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_mask(const BwdParams& p, hipStream_t st, int mg, int* out) {
    if (p.side_vec) return launch_vec<DT, HAS_BIAS, MASK_DT, true>(p, st, mg, out);
    return launch_vec<DT, HAS_BIAS, MASK_DT, false>(p, st, mg, out);
}

template <int DT>
static hipError_t launch_dt(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int mg, int* out) {
    if (has_bias) {
        if (mask_dt < 0) return launch_mask<DT, true, -1>(p, st, mg, out);
        if (mask_dt == FWA2_F32) return launch_mask<DT, true, FWA2_F32>(p, st, mg, out);
        return launch_mask<DT, true, DT>(p, st, mg, out);
    }
    if (mask_dt < 0) return launch_mask<DT, false, -1>(p, st, mg, out);
    if (mask_dt == FWA2_F32) return launch_mask<DT, false, FWA2_F32>(p, st, mg, out);
    return launch_mask<DT, false, DT>(p, st, mg, out);
}

// max_groups: workgroups per head and launch that the workspace has partial slots for.
hipError_t launch_backward_fused(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st,
                                 int max_groups, int* parts_out) {
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, st, max_groups, parts_out);
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, parts_out);
}

}  // namespace fwa2
