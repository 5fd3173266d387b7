// Backward, query side, for windows of up to 256 tokens: dq and the per-row
// terms of dlogit_scale from persistent workgroups that keep the bias tile
// resident in registers (longer windows use the streaming kernel in
// fwa2_bwd_dq.hip).
//
// Replaces the dq half of _bwd_kernel
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:84-564; the reference adds
// every key block's dq contribution into an fp32 buffer with atomics, :314).
//
// Same skeleton as the resident forward kernel: a workgroup belongs to one
// head, every wavefront owns 16 query rows and holds bias[h] * log2e - m for
// them in the register layout of the score accumulators (m = the row's logit
// bound s log2e + max bias2), K_hat (fp16) and V of the next unit land in LDS by
// DMA while the current unit is computed.  Per 32 keys:
//   S^T - m   = K_hat Q_hat^T        (fp16 MFMA, C operand = resident bias)
//   dP^T      = V dO^T               (input dtype MFMA, C operand = -delta)
//   dZ^T      = 2^(S^T - lse2) (dP^T - delta), rounded to fp16
//   dQ_hat^T += K_hat^T dZ^T         (fp16 MFMA, K_hat^T by transposing LDS reads)
// When the row bound is tight (bf16, moderate scale, masks that only remove
// keys) the factor w = 2^(m - lse2) is folded into dO and delta once per row,
// so that dZ^T = 2^acc * acc' costs one exp and one multiply per score.
// delta = rowsum(o * dO) is read from the buffer the key-side kernel wrote.
#include "fwa2_common.hpp"

// FWA2_HALF splits this translation unit for the build: 0 (default) the whole file; 1 everything except the
// fp16 instantiations, which it reaches through launch_backward_dq_resident_f16(); 2 the fp16 instantiations alone.
#ifndef FWA2_HALF
#define FWA2_HALF 0
#endif

namespace fwa2 {

constexpr int kDqSub = 2;    // 16-row query tiles per wavefront (see below)

// SUB = 16-row query tiles per wavefront.  With SUB = 2 a wavefront owns 32 query rows as two
// independent tiles that share every K / V operand it reads from LDS; a unit of 256 rows then takes
// 8 wavefronts of up to 256 registers instead of 16 of up to 128.
// MAPPED: rows are addressed through the window map (cyclic shift + window partition done here).
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MASKED, int SUB, bool MAPPED = false>
__global__ void __launch_bounds__(64 * NT / SUB) bwd_dq_resident_kernel(const BwdParams p) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    typedef ME MV8 __attribute__((ext_vector_type(8)));
    constexpr int ROWS = 16 * NT;
    constexpr int S = kLdsStride;
    constexpr int WR = 16 * SUB;          // rows per wavefront (queries owned, K / V rows staged)

    __shared__ __attribute__((aligned(16))) SE lds_K[2][ROWS * S];
    __shared__ __attribute__((aligned(16))) E lds_V[2][ROWS * S];
    __shared__ __attribute__((aligned(16))) E lds_rawK[ROWS * 32];   // landing area: unpadded 64-byte rows
    __shared__ __attribute__((aligned(16))) E lds_rawV[ROWS * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawQ[ROWS * 32];   // this wavefront's 16 query rows
    __shared__ __attribute__((aligned(16))) E lds_rawDO[ROWS * 32];
    __shared__ __attribute__((aligned(16))) float lds_rawLse[ROWS];  // lse and delta of the same rows
    __shared__ __attribute__((aligned(16))) float lds_rawDelta[ROWS];
    __shared__ uint8_t lds_live[kLiveCache];
    __shared__ uint16_t lds_list[kLiveCache];
    __shared__ int lds_count;
    __shared__ float lds_red[NT];

    const int N = p.n;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // uniform: lives in a scalar register
    const int l16 = lane & 15;
    const int g = lane >> 4;

    const int groups = p.dq_groups;
    const int h = blockIdx.x / groups;
    const int grp = blockIdx.x - h * groups;

    float s_true;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        s_true = expf(fminf(ls, kLn100));
    } else {
        s_true = p.default_scale;
    }
    const float scale2 = s_true * kLog2e;

    for (int i = tid; i < 2 * ROWS * S / 8; i += nthreads) {
        st8<SV8>(&lds_K[0][0] + i * 8, zero8<SV8>());
        st8<V8>(&lds_V[0][0] + i * 8, zero8<V8>());
    }
    for (int i = tid; i < ROWS * 32 / 8; i += nthreads) {
        st8<V8>(lds_rawK + i * 8, zero8<V8>());
        st8<V8>(lds_rawV + i * 8, zero8<V8>());
        st8<V8>(lds_rawQ + i * 8, zero8<V8>());
        st8<V8>(lds_rawDO + i * 8, zero8<V8>());
    }

    int qi[SUB], qc[SUB];
    bool qv[SUB];
#pragma unroll
    for (int u = 0; u < SUB; u++) {
        qi[u] = wave * WR + 16 * u + l16;
        qv[u] = qi[u] < N;
        qc[u] = min(qi[u], N - 1);
    }

    // ---- resident tile (see fwa2_fwd_resident.hip): acc0[u][2kp][i] <-> key 32kp + 8g + i,
    // acc0[u][2kp+1][i] <-> key 32kp + 8g + 4 + i of query tile u; (bias + mask) * log2e minus the
    // row bound m_fixed = s log2e + max_j (bias2 + mask2)[j] ----
    f32x4 acc0[SUB][NT];
    float m_fixed[SUB];
    auto build_tile = [&](int w) __attribute__((always_inline)) {
        // lane-derived offsets are re-materialised per call: hoisted out of the unit loop, the row
        // addresses of every key group would stay alive (and spilled) across all units
        int ln = lane;
        if (MASKED) asm volatile("" : "+v"(ln));
        const int g = ln >> 4;
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const E* brow = nullptr;
            const ME* mrow = nullptr;
            const int qrow = min(wave * WR + 16 * u + (ln & 15), N - 1);
            if (HAS_BIAS) brow = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qrow * p.bias_sn;
            if (MASKED) mrow = reinterpret_cast<const ME*>(p.mask) + w * p.mask_sw + (int64_t)qrow * p.mask_sn;
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
                    acc0[u][2 * kp + (j >> 2)][j & 3] = v[j];
                    mb = fmaxf(mb, v[j]);
                }
            }
            mb = col_max(mb);
            if (!(mb > -INFINITY)) mb = 0.f;        // every key of the row removed: nothing to bound
            m_fixed[u] = mb + scale2;
#pragma unroll
            for (int kt = 0; kt < NT; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc0[u][kt][i] -= m_fixed[u];
        }
    };
    // w = 2^(m - lse2) lies in [1/N, 2^(2 s log2e)]: it may be folded into dO when that cannot leave
    // the bf16 range
    const bool fold = (DT == FWA2_BF16) && (2.f * scale2 <= kGapLimit);

    // ---- which units belong to this launch (same dealing as in fwa2_fwd_resident.hip): the plain
    // launch deals the units of the unmasked windows out by rank; the MASKED launch deals the head's
    // workgroups out over the masked windows and rebuilds the tile per window ----
    const int nw = MASK_DT >= 0 ? p.n_windows : 1;
    const bool listed = MASK_DT >= 0 && p.mask_live != nullptr;      // the host drops the flags beyond kLiveCache
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
    int wi_step = 1, img0 = 0, img_step = 1, wi0 = grp;
    if (MASKED) {
        if (groups >= cnt && cnt > 0) {
            const int per = groups / cnt;         // workgroups per window
            wi0 = grp / per;                      // (>= cnt for the few left over: they idle)
            img0 = grp - wi0 * per;
            img_step = per;
            wi_step = cnt;                        // one window only
        } else {
            wi_step = groups;
        }
    }
    // the plain walk t -> t + groups without a division per unit: (img, wi) += (groups / cnt, groups % cnt)
    const int step_img = cnt > 0 ? groups / cnt : 0;
    const int step_wi = cnt > 0 ? groups - step_img * cnt : 0;
    struct Cursor { int wi, img; };
    auto valid = [&](const Cursor& c) -> bool { return MASKED ? c.wi < cnt : c.img < n_img; };
    auto first = [&]() -> Cursor {
        Cursor c;
        if (MASKED) { c.wi = wi0; c.img = img0; if (img0 >= n_img) c.wi = cnt; }
        else { c.img = cnt > 0 ? grp / cnt : n_img; c.wi = cnt > 0 ? grp - c.img * cnt : 0; }
        return c;
    };
    auto next = [&](Cursor c) -> Cursor {
        if (MASKED) {
            c.img += img_step;
            if (c.img >= n_img) { c.img = img0; c.wi += wi_step; }
        } else {
            c.img += step_img;
            c.wi += step_wi;
            if (c.wi >= cnt) { c.wi -= cnt; c.img += 1; }
        }
        return c;
    };
    auto unit_of = [&](const Cursor& c) -> int { return c.img * nw + window_at(c.wi); };

    // ---- per-unit fetch: the wavefront's WR rows of k, v (which it will stage) and of q, dO (its own
    // queries) by DMA, 16 rows per instruction; lse and delta of its queries in registers ----
    // issued by hand (see dma16_to_lds): the compiler would otherwise wait for the whole fetch in front of the
    // first transposing LDS read of every unit, which it cannot tell from the landing areas
    // The fetch of a unit comes in four parts (k rows with lse and delta, v, q, dO rows), each issued behind one of
    // the first four key groups of the unit before: requested in one burst right behind the barrier, the eighty
    // instructions of a workgroup queue up in the address unit for as long as two key groups take, with every
    // wavefront waiting in that queue and nothing to compute.
    auto fetch_part = [&](int b, int part) __attribute__((always_inline)) {
        // lane-derived offsets are re-materialised here: hoisted out of the unit loop they would occupy
        // a dozen registers for the whole kernel
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int fc8 = (ln & 3) * 8;
        const T4& t = part == 0 ? p.k : (part == 1 ? p.v : (part == 2 ? p.q : p.d_o));
        // unit start in scalar registers, rows as 32-bit byte offsets from it; landing addresses as integers from
        // the arrays' starts (the address of a __shared__ array is a compile-time constant; no pointer leaves the
        // LDS address space on the way)
        const void* unit = uniform_pointer(unit_ptr<MAPPED, E>(t, p.map, b, h));
        const uint32_t base = part == 0 ? lds_address(lds_rawK)
                                        : (part == 1 ? lds_address(lds_rawV) : (part == 2 ? lds_address(lds_rawQ) : lds_address(lds_rawDO)));
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const int row0 = wave * WR + 16 * u;
            const int frow = row0 + (ln >> 2);
            if (frow < N)
                dma16_to_lds(unit, row_byte_offset<E>(unit_row<MAPPED>(p.map, b, frow), t.sn, fc8),
                             base + (uint32_t)(row0 * 32 * sizeof(E)));
        }
        if (part == 0) {
            // lse and delta of the wavefront's rows, one row per lane
            const int q = wave * WR + ln;
            if (ln < WR && q < N) {
                dma4_to_lds(p.lse + b * p.lse_sb + h * p.lse_sh + q, lds_address(lds_rawLse + wave * WR));
                dma4_to_lds(p.delta + ((int64_t)b * p.heads + h) * p.delta_stride + q, lds_address(lds_rawDelta + wave * WR));
            }
        }
    };
    auto fetch = [&](int b) __attribute__((always_inline)) {
#pragma unroll
        for (int part = 0; part < 4; part++) fetch_part(b, part);
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const int fc8 = (lane & 3) * 8;
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const int frow = wave * WR + 16 * u + (lane >> 2);
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
        }
    };

    __syncthreads();
    Cursor c = first();
    int tile_wi = -1;                      // window index the resident tile was built for
    if (!MASKED) build_tile(0);
    if (valid(c)) {
        fetch(unit_of(c));
        stage(0);
    }
    __syncthreads();
    int cur = 0;
    float ds_acc = 0.f;        // sum over this lane's queries of q_hat . dq_hat

    while (valid(c)) {
        const int b = unit_of(c);
        const Cursor cn = next(c);
        const bool more = valid(cn);
        if (MASKED && c.wi != tile_wi) {
            build_tile(window_at(c.wi));
            tile_wi = c.wi;
        }

        // ---- this unit's operands out of the landed rows ----
        SV8 bq[SUB];
        V8 bd[SUB];
        f32x4 ndv[SUB], dqacc[SUB][2];
        float nl[SUB], inv[SUB];
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            // the rows landed before the previous unit's barrier (the first unit's before the one above)
            const V8 qcur = ld8<V8>(lds_rawQ + (wave * WR + 16 * u + l16) * 32 + 8 * g);
            const V8 docur = ld8<V8>(lds_rawDO + (wave * WR + 16 * u + l16) * 32 + 8 * g);
            const float lse_q = qv[u] ? lds_rawLse[wave * WR + 16 * u + l16] : -INFINITY;
            const float delta_q = qv[u] ? lds_rawDelta[wave * WR + 16 * u + l16] : 0.f;
            float x[8];
            unpack8(qcur, x);
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) ss += x[j] * x[j];
            ss = col_add(ss);
            inv[u] = inv_norm(ss);
            const float sc = scale2 * inv[u];
#pragma unroll
            for (int j = 0; j < 8; j++) bq[u][j] = (SE)(x[j] * sc);
            // fully masked row (lse = -inf): P = 0
            nl[u] = (lse_q == -INFINITY) ? -INFINITY : m_fixed[u] - lse_q * kLog2e;
            float nd;
            if (fold) {
                const float w = fast_exp2(nl[u]);
#pragma unroll
                for (int j = 0; j < 8; j++) bd[u][j] = (E)((float)docur[j] * w);
                nd = -delta_q * w;
                nl[u] = 0.f;
            } else {
                bd[u] = docur;
                nd = -delta_q;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) { dqacc[u][0][i] = 0.f; dqacc[u][1][i] = 0.f; ndv[u][i] = nd; }
        }
        const int b_next = more ? unit_of(cn) : 0;

        const SE* Kb = &lds_K[cur][0];
        const E* Vb = &lds_V[cur][0];

        auto group = [&](int kp, bool folded) __attribute__((always_inline)) {
            const int krow = 32 * kp + 8 * (l16 >> 2) + (l16 & 3);
            SV8 bz[SUB];
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const SV8 ak = ld8<SV8>(Kb + (krow + 4 * half) * S + 8 * g);
                const V8 av = ld8<V8>(Vb + (krow + 4 * half) * S + 8 * g);
#pragma unroll
                for (int u = 0; u < SUB; u++) {
                    f32x4 s = Elem<kScoreDT>::mfma16(ak, bq[u], acc0[u][2 * kp + half]);
                    const f32x4 dp = Elem<DT>::mfma16(av, bd[u], ndv[u]);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float e = folded ? fast_exp2(s[i]) : fast_exp2(s[i] + nl[u]);
                        bz[u][4 * half + i] = (SE)(e * dp[i]);
                    }
                }
            }
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4, so that this lane's accumulators hold d = 8g + 4dt + i
                const SE* klo = Kb + (32 * kp + 8 * g + (l16 >> 2)) * S + 8 * (l16 & 3) + 4 * dt;
                const SV8 akt = lds_tr8<kScoreDT>(klo, klo + 4 * S);
#pragma unroll
                for (int u = 0; u < SUB; u++) dqacc[u][dt] = Elem<kScoreDT>::mfma16(akt, bz[u], dqacc[u][dt]);
            }
        };
        auto body = [&](bool folded) __attribute__((always_inline)) {
#pragma unroll
            for (int kp = 0; kp < NT / 2; kp++) {
                progress_priority(kp, NT / 2);
                if (32 * kp < N) group(kp, folded);
                if (kp < 4 && more) fetch_part(b_next, kp);      // in flight while the rest of this unit is computed
            }
            if (more) {
#pragma unroll
                for (int part = NT / 2; part < 4; part++) fetch_part(b_next, part);     // tiles of fewer than four groups
            }
        };
        if (fold) body(true); else body(false);

        if (more) stage(cur ^ 1);     // before the stores below, so the wait covers only the fetch

        // ---- back through q / max(|q|, eps); q_hat . dq_hat is this row's share of dlogit_scale ----
        // q_hat is taken back from the fp16 score operand (q_hat s log2e), which is live anyway
        const float unscale = fast_rcp(scale2);
        int ln2 = lane;
        asm volatile("" : "+v"(ln2));
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            float qh[8];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                qh[j] = (float)bq[u][j] * unscale;
                dot += dqacc[u][j >> 2][j & 3] * qh[j];
            }
            dot = col_add(dot);
            const float proj = inv[u] < 0.5f / kNormEps ? dot : 0.f;      // |q| <= eps: no projection
            const float f = s_true * inv[u];
            const int q = wave * WR + 16 * u + (ln2 & 15);
            if (q < N) {
                E* dqrow = const_cast<E*>(row_ptr<MAPPED, E>(p.dq, p.map, b, h, q));
                V8 o8;
#pragma unroll
                for (int j = 0; j < 8; j++) o8[j] = (E)(f * (dqacc[u][j >> 2][j & 3] - qh[j] * proj));
                st8_stream<V8>(dqrow + 8 * (ln2 >> 4), o8);
                if (g == 0) ds_acc += dot;
            }
        }

        lds_barrier();         // next unit staged; everybody is done with the current buffers (the stores stay in flight)
        cur ^= 1;
        c = cn;
    }

    // ---- dlogit_scale: one partial per workgroup ----
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float wsum = wave_sum(ds_acc);
        if (lane == 0) lds_red[wave] = wsum;
        __syncthreads();
        if (tid == 0) {
            float tot = 0.f;
            for (int i = 0; i < (nthreads >> 6); i++) tot += lds_red[i];
            p.part_dscale[(int64_t)h * p.ds_parts + p.ds_slot0 + grp] = tot * s_true;
        }
    }
}

// ---- host side -----------------------------------------------------------------
#if FWA2_HALF != 2
int backward_dq_resident_supported(int n) { return n >= 1 && n <= 256; }
#endif

// Launches the kernel(s) and reports how many dscale partials per head they wrote.
// SUBP: 16-row query tiles per wavefront in the launch over the unmasked units; the masked launch always
// uses kDqSub (its tile rebuilds leave no room in 128 registers).
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, int SUBP = kDqSub, bool MAPPED = false>
static hipError_t launch_nt(BwdParams p, hipStream_t st, int max_groups, int* ds_parts_out) {
    constexpr int SUBM = kDqSub;
    static std::atomic<int> fit_plain_by_device[kFitDevices], fit_masked_by_device[kFitDevices];
    const int fit_plain = resident_per_cu_cached(bwd_dq_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, false, SUBP, MAPPED>,
                                                 64 * NT / SUBP, fit_plain_by_device);
    const int fit_masked =
        MASK_DT >= 0 ? resident_per_cu_cached(bwd_dq_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, true, SUBM, MAPPED>,
                                              64 * NT / SUBM, fit_masked_by_device)
                     : 1;
    auto groups_for = [&](int fit) {
        int groups = (p.cus * fit) / p.heads;
        if (groups < 1) groups = 1;
        if (groups > p.bw) groups = p.bw;
        if (groups > max_groups) groups = max_groups;
        return groups;
    };
    const bool two = MASK_DT >= 0 && p.mask_live != nullptr;
    const int g_plain = (MASK_DT < 0 || two) ? groups_for(fit_plain) : 0;
    const int g_masked = MASK_DT >= 0 ? groups_for(fit_masked) : 0;
    p.ds_parts = g_plain + g_masked;
    if (g_plain) {
        p.dq_groups = g_plain;
        p.ds_slot0 = 0;
        hipLaunchKernelGGL((bwd_dq_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, false, SUBP, MAPPED>), dim3(p.heads * g_plain),
                           dim3(64 * ((p.n + 16 * SUBP - 1) / (16 * SUBP))), 0, st, p);
    }
    if (g_masked) {
        p.dq_groups = g_masked;
        p.ds_slot0 = g_plain;
        hipLaunchKernelGGL((bwd_dq_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, true, SUBM, MAPPED>), dim3(p.heads * g_masked),
                           dim3(64 * ((p.n + 16 * SUBM - 1) / (16 * SUBM))), 0, st, p);
    }
    *ds_parts_out = p.ds_parts;
    return hipGetLastError();
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_mask(const BwdParams& p, hipStream_t st, int mg, int* out) {
    const int nt = p.n <= 64 ? 4 : (p.n <= 128 ? 8 : 16);
    if (p.map.nw > 0) {
        // windows of up to 64 tokens with a map go to the fused kernel, never here
        if (nt == 4) return hipErrorInvalidValue;
        if (p.side_vec || p.side_vec_rows) {
            if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, true, kDqSub, true>(p, st, mg, out);
            if (p.n <= 160) return launch_nt<DT, HAS_BIAS, MASK_DT, 10, true, 1, true>(p, st, mg, out);
            return launch_nt<DT, HAS_BIAS, MASK_DT, 16, true, kDqSub, true>(p, st, mg, out);
        }
        if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, false, kDqSub, true>(p, st, mg, out);
        if (p.n <= 160) return launch_nt<DT, HAS_BIAS, MASK_DT, 10, false, 1, true>(p, st, mg, out);
        return launch_nt<DT, HAS_BIAS, MASK_DT, 16, false, kDqSub, true>(p, st, mg, out);
    }
    if (p.side_vec || p.side_vec_rows) {
        if (nt == 4) return launch_nt<DT, HAS_BIAS, MASK_DT, 4, true>(p, st, mg, out);
        if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, true>(p, st, mg, out);
        // 129 .. 160 tokens: tiles of 160 keys (40 registers of resident bias per 16 rows instead of 64), and 16 rows
        // per wavefront, which gives nine or ten wavefronts instead of five
        if (p.n <= 160) return launch_nt<DT, HAS_BIAS, MASK_DT, 10, true, 1>(p, st, mg, out);
        return launch_nt<DT, HAS_BIAS, MASK_DT, 16, true>(p, st, mg, out);
    }
    if (nt == 4) return launch_nt<DT, HAS_BIAS, MASK_DT, 4, false>(p, st, mg, out);
    if (nt == 8) return launch_nt<DT, HAS_BIAS, MASK_DT, 8, false>(p, st, mg, out);
    if (p.n <= 160) return launch_nt<DT, HAS_BIAS, MASK_DT, 10, false, 1>(p, st, mg, out);
    return launch_nt<DT, HAS_BIAS, MASK_DT, 16, false>(p, st, mg, out);
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

// max_groups: workgroups per head and launch that the workspace has dscale slots for.
#if FWA2_HALF == 2
hipError_t launch_backward_dq_resident_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups,
                                           int* ds_parts_out) {
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, ds_parts_out);
}
#else
#if FWA2_HALF == 1
hipError_t launch_backward_dq_resident_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups,
                                           int* ds_parts_out);
#endif
hipError_t launch_backward_dq_resident(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st,
                                       int max_groups, int* ds_parts_out) {
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, st, max_groups, ds_parts_out);
#if FWA2_HALF == 1
    return launch_backward_dq_resident_f16(p, has_bias, mask_dt, st, max_groups, ds_parts_out);
#else
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, ds_parts_out);
#endif
}
#endif

}  // namespace fwa2
