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
// clamp of 100, masks with positive entries or fully masked rows) a first
// pass of score products alone finds the exact row maximum, and the same loop
// then runs against it.
//
// Per unit: K and V rows of the NEXT unit are fetched straight into an LDS
// landing area (global_load_lds, no registers held) before the tiles of the
// current one are computed; afterwards every wavefront normalises the 16 rows
// it fetched into the other half of a double buffer; one barrier per unit.
// Units whose window mask is live are walked by workgroups of their own, which run
// the MASKED form of the same body (resident tile = bias + the window's mask), so the
// common unmasked code carries no mask registers; both kinds of workgroup share one
// launch (fwd_resident_kernel below).
#include "fwa2_common.hpp"

// FWA2_HALF splits this translation unit for the build: 0 (default) the whole file; 1 everything except the
// fp16 instantiations, which it reaches through launch_forward_resident_f16(); 2 the fp16 instantiations alone.
#ifndef FWA2_HALF
#define FWA2_HALF 0
#endif

namespace fwa2 {

// NT = compile-time bound on the 16-key tiles of a unit (N <= 16 NT); the workgroup has
// ceil(N / 16) wavefronts.
// MASKED: this workgroup handles units whose window mask is live; the other units (or all, when
// there is no mask) go through the MASKED = false form.
// MAPPED: rows are addressed through the window map (cyclic shift + window partition done here).
// SUB: 16-row query tiles per wavefront.  Two tiles share every K / V operand read from LDS and leave the
// wavefront 256 registers, half as many wavefronts per workgroup.
// FULL: the window has exactly 16 NT tokens (64, 128, 256), so the window length is a compile-time constant and
// every bounds check, clamp and per-tile branch on it folds away.
// LDS address (a scalar) of a wavefront-uniform pointer into one of the shared_array() arrays: the low half of its flat address.
// (Cast to the LDS address space instead, the pointer would be checked for null at run time wherever the compiler
// has moved the cast behind a readfirstlane and no longer knows where the pointer came from.)
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)p);
}

// The walk of one workgroup (head h, workgroup grp of the `groups` its class has for that head) over its units.
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MASKED, bool MAPPED, int SUB = 1, bool FULL = false>
__device__ __forceinline__ void fwd_resident_body(const FwdParams& p, const int h, const int grp, const int groups) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    constexpr int ROWS = 16 * NT;
    constexpr int S = kLdsStride;
    constexpr int WR = 16 * SUB;          // rows per wavefront (queries owned, K / V rows staged)
    constexpr int IDS = WR + 16;          // bytes of the region landing area per wavefront: ids, then the value
    // Windows of up to 64 tokens come in problems small enough for the memory-side cache to matter: their outputs
    // are stored without the streaming hint, so the backward finds part of them there (the rows are still fetched
    // with it: from a cold cache plain fetches measured 12 % slower).
    constexpr bool STREAM = NT > 4;

    // the staged tiles, double-buffered
    SE (*lds_K)[ROWS * S] = reinterpret_cast<SE (*)[ROWS * S]>(shared_array<SE, 2 * ROWS * S, 0>());
    E (*lds_V)[ROWS * S] = reinterpret_cast<E (*)[ROWS * S]>(shared_array<E, 2 * ROWS * S, 1>());
    E* lds_rawK = shared_array<E, ROWS * 32, 2>();   // landing area: unpadded 64-byte rows
    E* lds_rawV = shared_array<E, ROWS * 32, 3>();
    E* lds_rawQ = shared_array<E, ROWS * 32, 4>();   // the wavefront's own query rows
    // REGIONS: the plain class also takes the windows whose mask has region form (RegionRecord): their mask term
    // comes out of one more MFMA per score tile, query-side operand in registers, key-side operand in lds_kop
    constexpr bool REGIONS = MASK_DT >= 0 && !MASKED;
    static_assert(kLdsStride >= 40 && kScoreDT == FWA2_F16,
                  "the key-side entries of the region product live in the 8 spare fp16 columns of the staged K rows");
    // landing area of the region record: per wavefront the ids of its rows, then the record's value ((NT / SUB) * IDS
    // bytes, which NT * 32 covers)
    uint8_t* lds_rawid = shared_array<uint8_t, (MASK_DT >= 0 ? NT * 32 : 32), 5>();
    uint8_t* lds_live = shared_array<uint8_t, kLiveCache, 6>();        // copy of the per-window mask flags
    uint16_t* lds_list = shared_array<uint16_t, kLiveCache, 7>();      // windows of this class, ascending
    int& lds_count = *shared_array<int, 4, 8>();

    const int N = FULL ? 16 * NT : p.n;
    // the per-group guards of the tile loops stay run-time tests even when N is a constant: they are what keeps
    // the scheduler to one key group at a time (merged into one block, the groups' loads are hoisted and spill)
    const int n_groups = p.n;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // uniform: lives in a scalar register
    const int l16 = lane & 15;       // query column inside the wavefront's 16 rows
    const int g = lane >> 4;         // accumulator rows 4g .. 4g+3, operand k-slots 8g .. 8g+7

    float scale2;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        scale2 = expf(fminf(ls, kLn100)) * kLog2e;
    } else {
        scale2 = p.default_scale * kLog2e;
    }

    // ---- which units belong to this workgroup's class.  With the mask flags at hand the windows of this
    // class (mask live or not) are listed once.
    //   plain class: the units of the listed windows (all units without a mask) are dealt out by
    //     their rank, so every workgroup of the head gets the same number of them;
    //   MASKED class: every workgroup of the head gets one stretch of the listed windows' units in
    //     window-major order, and the tile is rebuilt with the window's mask whenever a workgroup moves
    //     on to another window. ----
    const int nw = MASK_DT >= 0 ? p.n_windows : 1;
    const bool listed = MASK_DT >= 0 && p.mask_live != nullptr;      // the host drops the flags beyond kLiveCache
    if (listed) {
        for (int i = tid; i < nw; i += nthreads) lds_live[i] = p.mask_live[i];
        __syncthreads();
        if (wave == 0) {
            int c = 0;
            for (int base = 0; base < nw; base += 64) {
                const int w = base + lane;
                // a live window goes to the MASKED class unless its region record serves it here
                const bool in = w < nw && ((lds_live[w] != 0 && !(p.regions != nullptr && (lds_live[w] & 4))) == MASKED);
                const unsigned long long bal = __ballot(in);
                if (in) lds_list[c + __popcll(bal & ((1ull << lane) - 1ull))] = (uint16_t)w;
                c += __popcll(bal);
            }
            if (lane == 0) lds_count = c;
        }
        __syncthreads();
    }
    const int cnt = listed ? __builtin_amdgcn_readfirstlane(lds_count) : nw;    // windows of this class
    if (cnt == 0) return;                  // nothing for this class (every live window has region form, say)

    // rows of the staging buffers that no unit ever writes must read as zeros
    for (int i = tid; i < 2 * ROWS * S / 8; i += nthreads) {
        st8<SV8>(&lds_K[0][0] + i * 8, zero8<SV8>());
        st8<V8>(&lds_V[0][0] + i * 8, zero8<V8>());
    }
    for (int i = tid; i < ROWS * 32 / 8; i += nthreads) {
        st8<V8>(lds_rawK + i * 8, zero8<V8>());
        st8<V8>(lds_rawV + i * 8, zero8<V8>());
        st8<V8>(lds_rawQ + i * 8, zero8<V8>());
    }

    bool qv[SUB];
#pragma unroll
    for (int u = 0; u < SUB; u++) qv[u] = wave * WR + 16 * u + l16 < N;

    // ---- resident tile, log2 domain.  Keys are taken 32 at a time; of such a group this lane holds
    // keys 8g .. 8g+7: acc0[2kp][i] <-> key 32kp + 8g + i, acc0[2kp+1][i] <-> key 32kp + 8g + 4 + i
    // (so bias and mask rows are read 8 consecutive entries at a time).  The tile holds
    // (bias + mask) * log2e - m_fixed, m_fixed = s log2e + max_j (bias2 + mask2)[j] being an upper bound
    // of every logit of the row; the key that attains the maximum scores at least m_fixed - 2 s log2e. ----
    f32x4 acc0[SUB][NT];
    float m_fixed[SUB];
    float bias_range = 0.f;      // largest minus smallest bias (log2 domain) over this lane's rows
    auto build_tile = [&](int w) __attribute__((always_inline)) {
        // lane-derived offsets are re-materialised per call: hoisted out of the unit loop, the row
        // addresses of every key group would stay alive (and spilled) across all units
        int ln = lane;
        if (MASKED) asm volatile("" : "+v"(ln));
        const int g = ln >> 4;
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const int qrow = min(wave * WR + 16 * u + (ln & 15), N - 1);
            const E* brow = nullptr;
            const ME* mrow = nullptr;
            if (HAS_BIAS) brow = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qrow * p.bias_sn;
            if (MASKED) mrow = reinterpret_cast<const ME*>(p.mask) + w * p.mask_sw + (int64_t)qrow * p.mask_sn;
            float mb = -INFINITY, mn = INFINITY;
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
                    if (REGIONS && v[j] > -INFINITY) mn = fminf(mn, v[j]);
                }
            }
            mb = col_max(mb);
            if (REGIONS) bias_range = fmaxf(bias_range, mb - (-col_max(-mn)));
            if (!(mb > -INFINITY)) mb = 0.f;        // every key of the row removed: nothing to bound
            m_fixed[u] = mb + scale2;
#pragma unroll
            for (int kt = 0; kt < NT; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc0[u][kt][i] -= m_fixed[u];
        }
    };
    // the maximum-free softmax is used when the row bound cannot be further than this from the
    // largest logit (the same for every row of the head)
    const bool fast = (DT == FWA2_BF16) && (2.f * scale2 <= kGapLimit);

    const int n_img = p.bw / nw;
    auto window_at = [&](int wi) -> int {
        return listed ? __builtin_amdgcn_readfirstlane((int)lds_list[wi]) : wi;
    };
    // A cursor names one unit: (wi, img) = (index into the class's windows, image).
    //   plain:  rank t = img * cnt + wi walks t = grp, grp + groups, ...
    //   MASKED: the units in window-major order, t = wi * n_img + img, are cut into one stretch per workgroup
    //           (lengths differ by at most one), so a workgroup changes its window once or twice at most
    const int64_t units_m = (int64_t)cnt * n_img;
    const int t_first = MASKED ? (int)(units_m * grp / groups) : 0;
    const int t_count = MASKED ? (int)(units_m * (grp + 1) / groups) - t_first : 0;
    // the plain walk t -> t + groups without a division per unit: (img, wi) += (groups / cnt, groups % cnt)
    const int step_img = cnt > 0 ? groups / cnt : 0;
    const int step_wi = cnt > 0 ? groups - step_img * cnt : 0;
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
            c.img += step_img;
            c.wi += step_wi;
            if (c.wi >= cnt) { c.wi -= cnt; c.img += 1; }
        }
        return c;
    };
    auto unit_of = [&](const Cursor& c) -> int { return c.img * nw + window_at(c.wi); };
    // the region record of the cursor's window, or nullptr when the window has none (uniform)
    auto record_of = [&](const Cursor& c) -> const RegionRecord* {
        if (!REGIONS || p.regions == nullptr) return nullptr;
        const int w = window_at(c.wi);
        if (!(lds_live[w] & 4)) return nullptr;
        return reinterpret_cast<const RegionRecord*>(p.regions) + w;
    };

    // ---- per-unit fetch: every wavefront brings in the WR rows of K, V (which it will stage) and of Q (its own
    // queries) with that index, 16 rows per instruction (lane i lands at 16 i bytes from the base) ----
    auto fetch = [&](int b, const RegionRecord* rec) __attribute__((always_inline)) {
        // lane-derived offsets are re-materialised here: hoisted out of the unit loop they would be
        // spilled, and the reload would sit in front of every fetch
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int fc8 = (ln & 3) * 8;
        // unit starts in scalar registers, rows as 32-bit byte offsets from them
        const void* kunit = uniform_pointer(unit_ptr<MAPPED, E>(p.k, p.map, b, h));
        const void* vunit = uniform_pointer(unit_ptr<MAPPED, E>(p.v, p.map, b, h));
        const void* qunit = uniform_pointer(unit_ptr<MAPPED, E>(p.q, p.map, b, h));
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const int row0 = wave * WR + 16 * u;
            const int frow = row0 + (ln >> 2);
            if (frow < N) {
                const int pos = unit_row<MAPPED>(p.map, b, frow);
                dma16_to_lds(kunit, row_byte_offset<E>(pos, p.k.sn, fc8), lds_offset(lds_rawK + row0 * 32));
                dma16_to_lds(vunit, row_byte_offset<E>(pos, p.v.sn, fc8), lds_offset(lds_rawV + row0 * 32));
                dma16_to_lds(qunit, row_byte_offset<E>(pos, p.q.sn, fc8), lds_offset(lds_rawQ + row0 * 32));
            }
        }
        if (REGIONS && rec != nullptr && ln < 4 * SUB + 1) {    // the ids of this wavefront's rows, then the value
            const void* src = ln < 4 * SUB ? (const void*)(rec->id + wave * WR + 4 * ln) : (const void*)&rec->value;
            dma4_to_lds(src, lds_offset(lds_rawid + wave * IDS));
        }
    };
    // landing area -> tiles: K normalised and rounded to fp16, V as is (rows >= n stay zero)
    f16x4 qop[SUB];             // query-side operands of the region product for the unit staged last
#pragma unroll
    for (int u = 0; u < SUB; u++) qop[u] = f16x4{0, 0, 0, 0};
    auto stage = [&](int buf, const RegionRecord* rec) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // this wavefront's rows have landed
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int fc8 = (ln & 3) * 8;
        if (REGIONS && rec != nullptr) {
            const float value = *reinterpret_cast<const float*>(lds_rawid + wave * IDS + WR);
#pragma unroll
            for (int u = 0; u < SUB; u++) {
                qop[u] = region_query_operand(value * kLog2e, lds_rawid[wave * IDS + 16 * u + (ln & 15)], ln >> 4);
                if ((ln & 3) == 0)
                    st8<f16x8>(reinterpret_cast<_Float16*>(&lds_K[buf][(wave * WR + 16 * u + (ln >> 2)) * S + 32]),
                               region_key_entry(lds_rawid[wave * IDS + 16 * u + (ln >> 2)]));
            }
        }
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const int frow = wave * WR + 16 * u + (ln >> 2);
            const V8 kk = ld8<V8>(lds_rawK + frow * 32 + fc8);
            const V8 vv = ld8<V8>(lds_rawV + frow * 32 + fc8);
            float x[8];
            unpack8(kk, x);
            const float ss = quad_add(sumsq8(kk));
            const float inv = inv_norm(ss);
            SV8 kn;
#pragma unroll
            for (int j = 0; j < 8; j++) kn[j] = (SE)(x[j] * inv);
            st8<SV8>(&lds_K[buf][frow * S + fc8], kn);
            st8<V8>(&lds_V[buf][frow * S + fc8], vv);
        }
    };

    __syncthreads();                       // zero fill done
    Cursor c = first();
    int tile_wi = -1;                      // window index the resident tile was built for
    if (!MASKED) build_tile(0);
    // a region unit may skip the running maximum only if the row bound, which ignores the mask, cannot be
    // further from the largest logit than the gap limit: the key with the largest bias may be one the mask removes
    bool fast_reg = fast;
    if (REGIONS && p.regions != nullptr) fast_reg = fast && !__syncthreads_or(2.f * scale2 + bias_range > kGapLimit);
    if (valid(c)) {
        fetch(unit_of(c), record_of(c));
        stage(0, record_of(c));
    }
    __syncthreads();
    int cur = 0;

    while (valid(c)) {
        const int b = unit_of(c);
        const Cursor cn = next(c);
        const bool more = valid(cn);
        if (MASKED && c.wi != tile_wi) {
            build_tile(window_at(c.wi));
            tile_wi = c.wi;
        }
        // ---- Q operands: normalise, fold s log2e, round to fp16 ----
        SV8 bq[SUB];
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            // the rows landed before the previous unit's barrier (the first unit's before the one above)
            const V8 qq = ld8<V8>(lds_rawQ + (wave * WR + 16 * u + l16) * 32 + 8 * g);
            float x[8];
            unpack8(qq, x);
            const float ss = col_add(sumsq8(qq));
            const float sc = scale2 * inv_norm(ss);
#pragma unroll
            for (int j = 0; j < 8; j++) bq[u][j] = (SE)(x[j] * sc);
        }
        const RegionRecord* rec = record_of(c);
        const RegionRecord* rec_next = more ? record_of(cn) : nullptr;
        const bool reg = REGIONS && rec != nullptr;
        if (more) fetch(unit_of(cn), rec_next);      // in flight while this unit is computed

        const SE* Kb = &lds_K[cur][0];
        const E* Vb = &lds_V[cur][0];
        f32x4 oacc[SUB][2];
        f32x4 lacc[SUB];
        float m_run[SUB];      // exact-maximum path: row maximum relative to m_fixed
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            m_run[u] = 0.f;
#pragma unroll
            for (int i = 0; i < 4; i++) { oacc[u][0][i] = 0.f; oacc[u][1][i] = 0.f; lacc[u][i] = 0.f; }
        }

        // scores of keys 32 kp .. 32 kp + 31: MFMA tile A holds keys 8r/4 + r%4 in its rows r, tile B
        // the keys 4 further on, so that this lane's 8 values are keys 8g .. 8g+7 of the group; the two K
        // operands serve every query tile of the wavefront
        auto scores = [&](int kp, f32x4 (&s0)[SUB], f32x4 (&s1)[SUB], bool with_regions) __attribute__((always_inline)) {
            const int krow = 32 * kp + 8 * (l16 >> 2) + (l16 & 3);
            const SV8 a0 = ld8<SV8>(Kb + krow * S + 8 * g);
            const SV8 a1 = ld8<SV8>(Kb + (krow + 4) * S + 8 * g);
#pragma unroll
            for (int u = 0; u < SUB; u++) {
                s0[u] = Elem<kScoreDT>::mfma16(a0, bq[u], acc0[u][2 * kp]);
                s1[u] = Elem<kScoreDT>::mfma16(a1, bq[u], acc0[u][2 * kp + 1]);
            }
            if (REGIONS && with_regions) {
                // the lane's offset is derived again here: hoisted out of the unit loop, the eight addresses
                // (one per key group) would be spilled
                int ln = lane;
                asm volatile("" : "+v"(ln));
                const _Float16* ko = reinterpret_cast<const _Float16*>(Kb) +
                                     (32 * kp + 2 * (ln & 12) + (ln & 3)) * S + 32 + ((ln >> 2) & 4);
                // read by hand: the compiler cannot tell these reads from the landing areas the fetch of the next
                // unit is still writing, and would wait for that fetch in front of every one of them
                f16x4 k0, k1;
                asm volatile("ds_read_b64 %0, %2\n\tds_read_b64 %1, %2 offset:%3\n\ts_waitcnt lgkmcnt(0)"
                             : "=&v"(k0), "=&v"(k1)
                             : "v"((uint32_t)(uintptr_t)ko), "n"(4 * S * 2));
#pragma unroll
                for (int u = 0; u < SUB; u++) {
                    s0[u] = region_mfma(k0, qop[u], s0[u]);
                    s1[u] = region_mfma(k1, qop[u], s1[u]);
                }
            }
        };
        // The row sum comes out of a third MFMA against a tile of ones, i.e. it sums the ROUNDED P~ values
        // that also enter the product with V: o is then an exact convex combination of V rows, and the sum
        // costs no VALU work.  The transposed V operands serve every query tile of the wavefront.
        V8 ones;
#pragma unroll
        for (int j = 0; j < 8; j++) ones[j] = (E)1.0f;
        auto pv = [&](int kp, const f32x4 (&s0)[SUB], const f32x4 (&s1)[SUB]) __attribute__((always_inline)) {
            V8 bp[SUB];
#pragma unroll
            for (int u = 0; u < SUB; u++) {
#pragma unroll
                for (int i = 0; i < 4; i++) { bp[u][i] = (E)s0[u][i]; bp[u][4 + i] = (E)s1[u][i]; }
                lacc[u] = Elem<DT>::mfma16(ones, bp[u], lacc[u]);
            }
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4: this lane's accumulators hold d = 8g + 4dt + i
                const E* vlo = Vb + (32 * kp + 8 * g + (l16 >> 2)) * S + 8 * (l16 & 3) + 4 * dt;
                const V8 av = lds_tr8<DT>(vlo, vlo + 4 * S);
#pragma unroll
                for (int u = 0; u < SUB; u++) oacc[u][dt] = Elem<DT>::mfma16(av, bp[u], oacc[u][dt]);
            }
        };

        // the loop in two copies, so that units without a region record run exactly the code they would run
        // if there were no such units
        auto tiles = [&](bool use_fast, bool with_regions) __attribute__((always_inline)) {
            if (use_fast) {
#pragma unroll
                for (int kp = 0; kp < NT / 2; kp++) {
                    if (32 * kp < n_groups) {
                        progress_priority(kp, NT / 2);
                        f32x4 s0[SUB], s1[SUB];
                        scores(kp, s0, s1, with_regions);
#pragma unroll
                        for (int u = 0; u < SUB; u++)
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                s0[u][i] = fast_exp2(s0[u][i]);
                                s1[u][i] = fast_exp2(s1[u][i]);
                            }
                        pv(kp, s0, s1);
                    }
                }
            } else {
                // fp16 (P would underflow against a mere bound) or a very large scale: the exact row maximum
                // first, from a pass of score products alone; the matrix pipe has the room, and the second pass
                // then needs no running maximum, no rescaling of o and no VALU row sum
                float bm[SUB];
#pragma unroll
                for (int u = 0; u < SUB; u++) bm[u] = -INFINITY;
#pragma unroll
                for (int kp = 0; kp < NT / 2; kp++) {
                    if (32 * kp < n_groups) {
                        f32x4 s0[SUB], s1[SUB];
                        scores(kp, s0, s1, with_regions);
#pragma unroll
                        for (int u = 0; u < SUB; u++) {
                            bm[u] = fmaxf(bm[u], fmaxf(fmaxf(s0[u][0], s0[u][1]), fmaxf(s0[u][2], s0[u][3])));
                            bm[u] = fmaxf(bm[u], fmaxf(fmaxf(s1[u][0], s1[u][1]), fmaxf(s1[u][2], s1[u][3])));
                        }
                    }
                }
                float m_use[SUB];
#pragma unroll
                for (int u = 0; u < SUB; u++) {
                    m_run[u] = col_max(bm[u]);
                    m_use[u] = (m_run[u] == -INFINITY) ? 0.f : m_run[u];
                }
#pragma unroll
                for (int kp = 0; kp < NT / 2; kp++) {
                    if (32 * kp < n_groups) {
                        f32x4 s0[SUB], s1[SUB];
                        scores(kp, s0, s1, with_regions);
#pragma unroll
                        for (int u = 0; u < SUB; u++)
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                s0[u][i] = fast_exp2(s0[u][i] - m_use[u]);
                                s1[u][i] = fast_exp2(s1[u][i] - m_use[u]);
                            }
                        pv(kp, s0, s1);
                    }
                }
            }
        };
        if (REGIONS && reg) tiles(fast_reg, true);
        else tiles(fast, false);

        if (more) stage(cur ^ 1, rec_next);     // before the stores below, so the wait covers only the fetch
        // ---- normalise, write o (input dtype) and lse (natural log, fp32) ----
        int ln2 = lane;
        asm volatile("" : "+v"(ln2));
#pragma unroll
        for (int u = 0; u < SUB; u++) {
            const float l_tot = lacc[u][0];
            const float inv_l = l_tot > 0.f ? fast_rcp(l_tot) : 0.f;
            const int oq = wave * WR + 16 * u + (ln2 & 15);
            if (qv[u]) {
                E* orow = const_cast<E*>(row_ptr<MAPPED, E>(p.o, p.map, b, h, oq));
                V8 ov;
#pragma unroll
                for (int j = 0; j < 8; j++) ov[j] = (E)(oacc[u][j >> 2][j & 3] * inv_l);
                st8_stream<V8, E, STREAM>(orow + 8 * (ln2 >> 4), ov);
                if ((ln2 >> 4) == 0) {
                    const float lse = l_tot > 0.f ? (m_fixed[u] + m_run[u] + fast_log2(l_tot)) * kLn2 : -INFINITY;
                    p.lse[b * p.lse_sb + h * p.lse_sh + oq] = lse;
                }
            }
        }

        lds_barrier();         // next unit staged; everybody is done with the current buffers (the stores stay in flight)
        cur ^= 1;
        c = cn;
    }
}

// One launch for all the units of a call.  Without a mask every workgroup runs the plain body.  With one, the
// workgroups of a head are split between the two classes of windows in proportion to their numbers (every window has
// the same number of images): the first ones run the plain body over the windows whose mask is all zero (or has
// region form, where the records are in use), the others the MASKED body over the rest, side by side in one grid, so
// the chip sees one ramp and one tail.  Without mask flags every window counts as masked.
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MAPPED, int SUB, bool FULL>
__global__ void __launch_bounds__(64 * NT / SUB) fwd_resident_kernel(const FwdParams p) {
    static_assert(MASK_DT < 0 || SUB == 1, "both classes of a masked call run one query tile per wavefront");
    const int h = blockIdx.x / p.groups;
    const int grp = blockIdx.x - h * p.groups;
#define FWA2_FWD_BODY(M, G0, GN) \
    fwd_resident_body<DT, HAS_BIAS, MASK_DT, NT, VEC, M, MAPPED, SUB, FULL>(p, h, G0, GN)
    if constexpr (MASK_DT < 0) {
        FWA2_FWD_BODY(false, grp, p.groups);
    } else {
        // windows of the MASKED class: a live mask that no region record serves here (every window without flags)
        const int nw = p.n_windows;
        int n_masked = nw;
        if (p.mask_live != nullptr) {
            const int lane = threadIdx.x & 63;
            n_masked = 0;
            for (int base = 0; base < nw; base += 64) {
                const int w = base + lane;
                const uint8_t f = w < nw ? p.mask_live[w] : (uint8_t)0;
                n_masked += __popcll(__ballot(f != 0 && !(p.regions != nullptr && (f & 4))));
            }
            n_masked = __builtin_amdgcn_readfirstlane(n_masked);
        }
        if (n_masked == 0) {
            FWA2_FWD_BODY(false, grp, p.groups);
        } else if (n_masked == nw) {
            FWA2_FWD_BODY(true, grp, p.groups);
        } else if (p.groups < 2) {
            // a single workgroup per head: one class after the other
            FWA2_FWD_BODY(false, 0, 1);
            __syncthreads();
            FWA2_FWD_BODY(true, 0, 1);
        } else {
            int g_masked = (int)(((int64_t)p.groups * n_masked + nw / 2) / nw);
            g_masked = g_masked < 1 ? 1 : (g_masked > p.groups - 1 ? p.groups - 1 : g_masked);
            const int g_plain = p.groups - g_masked;
            if (grp < g_plain) FWA2_FWD_BODY(false, grp, g_plain);
            else FWA2_FWD_BODY(true, grp - g_plain, g_masked);
        }
    }
#undef FWA2_FWD_BODY
}

// ---- host side -----------------------------------------------------------------
#if FWA2_HALF != 2
int forward_resident_supported(int n) { return n >= 1 && n <= 256; }
#endif

#ifndef FWA2_FWD_SUB
#define FWA2_FWD_SUB 1
#endif
constexpr int kFwdSub = FWA2_FWD_SUB;    // 16-row query tiles per wavefront of the 256-token forward (calls without a mask)
constexpr int kRegionMaxImages = 32;     // images per window up to which region records are used (see launch_map)

// SUBP: 16-row query tiles per wavefront of a call without a mask (a masked call keeps one: its tile rebuilds want
// the registers, and both classes share the workgroup size).
template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC, bool MAPPED, int SUBP, bool FULL>
static hipError_t launch_map(FwdParams p, hipStream_t st) {
    constexpr int SUB = MASK_DT < 0 ? SUBP : 1;
    const int waves = (p.n + 16 * SUB - 1) / (16 * SUB);
    // the runtime's figure is for full groups; smaller groups only fit better
    static std::atomic<int> fit_by_device[kFitDevices];
    const int fit = resident_per_cu_cached(fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, MAPPED, SUB, FULL>, 64 * NT / SUB,
                                           fit_by_device);
    int groups = (p.cus * fit) / p.heads;
    if (groups < 1) groups = 1;
    if (groups > p.bw) groups = p.bw;
    p.groups = groups;
    // Windows whose mask has region form can ride with the unmasked ones, which saves the masked class its tile
    // rebuilds: measured on the 256-token benchmark shape (as two launches) that is 25 % of the forward time at 2
    // images per window, 8 % at 8, nothing at 32 and a loss of 3 % at 64.
    if (p.regions != nullptr && p.bw / p.n_windows > kRegionMaxImages) p.regions = nullptr;
    hipLaunchKernelGGL((fwd_resident_kernel<DT, HAS_BIAS, MASK_DT, NT, VEC, MAPPED, SUB, FULL>), dim3(p.heads * p.groups),
                       dim3(64 * waves), 0, st, p);
    return hipGetLastError();
}

template <int DT, bool HAS_BIAS, int MASK_DT, int NT, bool VEC>
static hipError_t launch_nt(const FwdParams& p, hipStream_t st) {
    constexpr int SUBP = NT == 16 ? kFwdSub : 1;       // the 256-token form; smaller tiles keep 16 rows per wavefront
    // whole tiles of 16 tokens get the form with a compile-time window length; such windows have rows of a
    // multiple of 8 entries, so they only exist with VEC
    if constexpr (VEC) {
        if (p.n == 16 * NT) {
            if (p.map.nw > 0) return launch_map<DT, HAS_BIAS, MASK_DT, NT, VEC, true, SUBP, true>(p, st);
            return launch_map<DT, HAS_BIAS, MASK_DT, NT, VEC, false, SUBP, true>(p, st);
        }
    }
    if (p.map.nw > 0) return launch_map<DT, HAS_BIAS, MASK_DT, NT, VEC, true, SUBP, false>(p, st);
    return launch_map<DT, HAS_BIAS, MASK_DT, NT, VEC, false, SUBP, false>(p, st);
}

template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_mask(const FwdParams& p, hipStream_t st) {
    const int nt = p.n <= 64 ? 4 : (p.n <= 128 ? 8 : 16);
    if (p.side_vec || p.side_vec_rows) {
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

#if FWA2_HALF == 2
hipError_t launch_forward_resident_f16(const FwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st);
}
#else
#if FWA2_HALF == 1
hipError_t launch_forward_resident_f16(const FwdParams& p, bool has_bias, int mask_dt, hipStream_t st);
#endif
hipError_t launch_forward_resident(const FwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    if (dtype == FWA2_BF16) return launch_dt<FWA2_BF16>(p, has_bias, mask_dt, st);
#if FWA2_HALF == 1
    return launch_forward_resident_f16(p, has_bias, mask_dt, st);
#else
    return launch_dt<FWA2_F16>(p, has_bias, mask_dt, st);
#endif
}
#endif

}  // namespace fwa2
