// Head dimensions other than 32 (any multiple of 8 up to 128): forward and backward for gfx950.
//
// The reference pads the head dimension to a power of two of at least 16 and supports up to 128
// (flash_win_attn_v2/kernels/attn_kernel_forward.py:267, 298); every configuration it benchmarks uses 32,
// which the tuned kernels of this library cover.  The kernels here restore the rest of that contract with
// one plain skeleton instead of five tuned ones: no register-resident bias, no persistent workgroups, no
// LDS DMA (the rows of the next step are fetched into registers while this step computes).
//
// One skeleton, four modes.  A workgroup of four wavefronts works on one (batch*window, head) unit and 64
// "owner" rows, 16 per wavefront, one per lane column (lane % 16); it walks over the "other" rows in steps
// of 32, which all four wavefronts share through LDS:
//
//   FWD    owner = queries, other = keys:     online softmax, O^T += V^T P^T
//   DQ     owner = queries, other = keys:     delta = rowsum(o * dO), dQ^^T += K^^T dZ^T; per-row dscale terms
//   DKV    owner = keys,    other = queries:  dK^^T += Q^^T dZ, dV^T += dO^T P
//   DBIAS  owner = queries, other = 32 keys:  loops over the units of a group, sums dZ per (query, key);
//          only for windows of more than 256 tokens: up to there DQ walks a group of units itself and
//          keeps the dZ sums of its 16 x N strip in registers
//
// Every score tile is v_mfma_f32_16x16x32 with the other rows as A rows and the owner rows as B columns, so
// a lane holds, for its owner row, the 8 consecutive other rows 8g .. 8g+7 (g = lane / 16) of the step: the
// rows of the two 16-row MFMA tiles are interleaved (tile a holds rows 8(r/4) + r%4 + 4a) to make them
// consecutive.  Those 8 values are directly the B operand (k = other rows) of the products that contract
// over the other rows; their A operands, the transposes of the staged tiles, come from row-major LDS with
// ds_read_b64_tr_b16, one 32-column slab of the head dimension at a time.
//
// Numerics follow the tuned kernels: q^ and k^ are rounded to fp16 for the score product (also for bf16
// inputs), scores live in the log2 domain, everything between the matrix products is fp32, P and dZ are
// rounded (P to the input dtype, dZ to fp16) for the second products.  Nothing is accumulated with atomics:
// dbias goes through per-group partial tiles and dlogit_scale through per-row terms, both summed in a fixed
// order by small reduction kernels, so gradients are bit-reproducible here too.
#include <string.h>

#include "fwa2_common.hpp"

namespace fwa2 {

enum { G_FWD = 0, G_DQ = 1, G_DKV = 2, G_DBIAS = 3 };

struct GenParams {
    T4 q, k, v, o, d_o, dq, dk, dv;
    WinMap map;           // nw == 0: off
    const void* logit_scale;
    int scale_kind;
    float default_scale;
    const void* bias;
    int64_t bias_sh, bias_sn;
    const void* mask;
    int64_t mask_sw, mask_sn;
    int mask_f32;
    int n_windows;
    const uint8_t* mask_live;   // [n_windows] 0 = the window's mask is all zero; nullptr = unknown
    int side_vec;               // rows of bias and mask may be read with 16-byte loads and n % 8 == 0
    float* lse;
    int64_t lse_sb, lse_sh;
    int bw, heads, n, nk, d;   // n queries, nk keys per unit
    float* delta;         // [BW * H, row_pad] rowsum(o * dO), written by DQ, read by DKV and DBIAS
    float* dscale_rows;   // [BW * H, row_pad] q^ . dq^ of every query row, written by DQ
    int row_pad;
    float* part_dbias;    // [groups, H, N, N] fp32
    int groups;           // unit groups of the DBIAS launch (group g sums units g, g + groups, ...)
    void* dbias;          // [H, N, N] input dtype
    void* dscale;         // [H] input dtype
};

// WITH_DB (DQ only, windows of up to 256 tokens): the workgroup walks the units of a group and also sums
// dZ per (query, key) in registers, which saves the separate DBIAS pass.
template <int DT, int D, int MODE, bool WITH_DB = false>
__global__ void __launch_bounds__(256) generic_kernel(const GenParams p) {
    static_assert(!WITH_DB || MODE == G_DQ, "dbias rides on the dq pass only");
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    constexpr int S = D + 8;         // LDS row stride in elements
    constexpr int KS = D / 32;       // 32-wide slabs of the head dimension
    constexpr int CH = D / 8;        // 16-byte chunks per row
    constexpr bool OWNER_IS_KEY = MODE == G_DKV;

    __shared__ __attribute__((aligned(16))) SE t0[32 * S];   // other rows, normalised (k^ or q^)
    __shared__ __attribute__((aligned(16))) E t1[32 * S];    // other rows of v (or dO)
    __shared__ float s_lse2[32], s_delta[32];                // DKV: lse log2(e) and delta of the other rows
    constexpr int AS = 68;                                   // row stride of s_add
    __shared__ float s_add[MODE == G_DKV ? 32 * AS : 1];     // DKV: (bias + mask) log2(e), [other query][owner key]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int d = p.d;
    const int NO = OWNER_IS_KEY ? p.nk : p.n;    // owner rows of a unit
    const int NX = OWNER_IS_KEY ? p.n : p.nk;    // other rows of a unit
    const int NQ = p.n, NKEY = p.nk;
    const int chunks = (NO + 63) / 64;
    const int kblocks = (NX + 31) / 32;

    int idx = blockIdx.x, kb = 0, grp = 0, b0;
    if (MODE == G_DBIAS) {
        kb = idx % kblocks;
        idx /= kblocks;
    }
    const int own0 = 64 * (idx % chunks);
    idx /= chunks;
    const int h = idx % p.heads;
    idx /= p.heads;
    if (MODE == G_DBIAS || WITH_DB) { grp = idx; b0 = grp; } else { b0 = idx; }

    const int own = own0 + 16 * wave + l16;     // owner row of this lane's column
    const bool own_ok = own < NO;

    float scale2, scale_nat;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        scale_nat = expf(fminf(ls, kLn100));
    } else {
        scale_nat = p.default_scale;
    }
    scale2 = scale_nat * kLog2e;

    // row `row` of unit b; with a window map the unit's rows lie scattered over the token grid
    const bool mapped = p.map.nw > 0;
    auto rowp = [&](const T4& t, int b, int row) -> const E* {
        const int64_t off = mapped ? row_off<true>(t, p.map, b, h, row) : row_off<false>(t, p.map, b, h, row);
        return reinterpret_cast<const E*>(t.ptr) + off;
    };

    // ---- owner rows: B operands of the score products, one row per lane column ----
    SV8 bs[KS];          // q^ (k^ for DKV), columns 32 s + 8 g .. + 7
    V8 bp[KS];           // dO (v for DKV), same columns; unused by FWD
    float own_inv = 0.f, own_lse2 = 0.f, own_delta = 0.f;
    auto load_owner = [&](int b) __attribute__((always_inline)) {
        const T4& ts = OWNER_IS_KEY ? p.k : p.q;
        float x[KS][8];
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const int col = 32 * s + 8 * g;
            V8 a = zero8<V8>();
            if (own_ok && col < d) a = ld8<V8>(rowp(ts, b, own) + col);
            unpack8(a, x[s]);
#pragma unroll
            for (int j = 0; j < 8; j++) ss += x[s][j] * x[s][j];
        }
        ss = col_add(ss);
        own_inv = inv_norm(ss);
#pragma unroll
        for (int s = 0; s < KS; s++)
#pragma unroll
            for (int j = 0; j < 8; j++) bs[s][j] = (SE)(x[s][j] * own_inv);
        if (MODE != G_FWD) {
            const T4& tp = OWNER_IS_KEY ? p.v : p.d_o;
            float dl = 0.f;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const int col = 32 * s + 8 * g;
                bp[s] = zero8<V8>();
                if (own_ok && col < d) {
                    bp[s] = ld8<V8>(rowp(tp, b, own) + col);
                    if (MODE == G_DQ) {
                        const V8 ov = ld8<V8>(rowp(p.o, b, own) + col);
#pragma unroll
                        for (int j = 0; j < 8; j++) dl += (float)bp[s][j] * (float)ov[j];
                    }
                }
            }
            const int64_t ro = ((int64_t)b * p.heads + h) * p.row_pad + own;
            if (MODE == G_DQ) {
                own_delta = col_add(dl);
                if (g == 0 && own_ok) p.delta[ro] = own_delta;
            }
            if (MODE == G_DBIAS) own_delta = own_ok ? p.delta[ro] : 0.f;
            if (MODE == G_DQ || MODE == G_DBIAS)
                own_lse2 = own_ok ? p.lse[b * p.lse_sb + h * p.lse_sh + own] * kLog2e : 0.f;
        }
    };

    // ---- 32 other rows starting at o0: fetch() brings this thread's share into registers (issued a step
    // ahead, so the loads fly during the matrix work), commit() normalises and stores it to LDS ----
    constexpr int NCH = (32 * CH + 255) / 256;     // 16-byte chunks of each tile per thread
    struct Staged {
        V8 a[NCH], bb[NCH];
        float add[8];          // DKV: (bias + mask) of one query against 8 owner keys
        float lse2, delta;     // DKV: of other row tid (threads 0 .. 31)
    };
    auto fetch = [&](int b, int o0, Staged& st) __attribute__((always_inline)) {
        const T4& ta = OWNER_IS_KEY ? p.q : p.k;
        const T4& tb = OWNER_IS_KEY ? p.d_o : p.v;
#pragma unroll
        for (int u = 0; u < NCH; u++) {
            const int c = tid + 256 * u;
            const int r = c / CH, c8 = (c % CH) * 8;
            const int row = o0 + r;
            st.a[u] = zero8<V8>();
            st.bb[u] = zero8<V8>();
            if (c < 32 * CH && row < NX && c8 < d) {
                st.a[u] = ld8<V8>(rowp(ta, b, row) + c8);
                st.bb[u] = ld8<V8>(rowp(tb, b, row) + c8);
            }
        }
        if (MODE == G_DKV) {
            // (bias + mask) of the 32 staged queries against the 64 owner keys, read along the rows of the
            // tables (the owner lanes need a column of them)
            const int r = tid >> 3, c8 = (tid & 7) * 8;
            const int qi = o0 + r, k0 = own0 + c8;
            const int w = b % p.n_windows;
            const bool mask_on = p.mask && (!p.mask_live || p.mask_live[w] != 0);
            float* add = st.add;
#pragma unroll
            for (int j = 0; j < 8; j++) add[j] = 0.f;
            if (qi < NQ) {
                const E* bptr = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)qi * p.bias_sn + k0;
                const int64_t mo = w * p.mask_sw + (int64_t)qi * p.mask_sn + k0;
                if (p.side_vec) {
                    if (k0 < NKEY) {
                        if (p.bias) {
                            const V8 bv = ld8<V8>(bptr);
#pragma unroll
                            for (int j = 0; j < 8; j++) add[j] += (float)bv[j];
                        }
                        if (mask_on && p.mask_f32) {
                            const f32x4 m0 = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mo);
                            const f32x4 m1 = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mo + 4);
#pragma unroll
                            for (int j = 0; j < 4; j++) { add[j] += m0[j]; add[4 + j] += m1[j]; }
                        } else if (mask_on) {
                            const V8 mv = ld8<V8>(reinterpret_cast<const E*>(p.mask) + mo);
#pragma unroll
                            for (int j = 0; j < 8; j++) add[j] += (float)mv[j];
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        if (k0 + j < NKEY) {
                            if (p.bias) add[j] += (float)bptr[j];
                            if (mask_on)
                                add[j] += p.mask_f32 ? reinterpret_cast<const float*>(p.mask)[mo + j]
                                                     : (float)reinterpret_cast<const E*>(p.mask)[mo + j];
                        }
                    }
                }
            }
            st.lse2 = 0.f;
            st.delta = 0.f;
            if (tid < 32 && o0 + tid < NX) {
                const int row = o0 + tid;
                st.lse2 = p.lse[b * p.lse_sb + h * p.lse_sh + row] * kLog2e;
                st.delta = p.delta[((int64_t)b * p.heads + h) * p.row_pad + row];
            }
        }
    };
    auto commit = [&](const Staged& st) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NCH; u++) {
            const int c = tid + 256 * u;
            if (c < 32 * CH) {       // whole aligned groups of CH lanes take part, so the shuffles stay inside
                const int r = c / CH, c8 = (c % CH) * 8;
                float x[8];
                unpack8(st.a[u], x);
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < 8; j++) ss += x[j] * x[j];
#pragma unroll
                for (int off = CH / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
                const float inv = inv_norm(ss);
                SV8 w;
#pragma unroll
                for (int j = 0; j < 8; j++) w[j] = (SE)(x[j] * inv);
                st8<SV8>(t0 + r * S + c8, w);
                st8<V8>(t1 + r * S + c8, st.bb[u]);
            }
        }
        if (MODE == G_DKV) {
            const int r = tid >> 3, c8 = (tid & 7) * 8;
#pragma unroll
            for (int j = 0; j < 8; j++) s_add[r * AS + c8 + j] = st.add[j] * kLog2e;
            if (tid < 32) {
                s_lse2[tid] = st.lse2;
                s_delta[tid] = st.delta;
            }
        }
    };

    // ---- one step: scores (and dP) of the staged rows against the owner rows ----
    // z2[j], dpv[j]: other row o0 + 8 g + j against owner row `own`; ok[j]: both rows exist
    auto tile = [&](int b, int o0, float* z2, float* dpv, bool* ok) __attribute__((always_inline)) {
        f32x4 sa[2], da[2];
#pragma unroll
        for (int a = 0; a < 2; a++) {
#pragma unroll
            for (int i = 0; i < 4; i++) { sa[a][i] = 0.f; da[a][i] = 0.f; }
            const int ar = 8 * (l16 >> 2) + (l16 & 3) + 4 * a;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const SV8 a0 = ld8<SV8>(t0 + ar * S + 32 * s + 8 * g);
                sa[a] = Elem<kScoreDT>::mfma16(a0, bs[s], sa[a]);
                if (MODE != G_FWD) {
                    const V8 a1 = ld8<V8>(t1 + ar * S + 32 * s + 8 * g);
                    da[a] = Elem<DT>::mfma16(a1, bp[s], da[a]);
                }
            }
        }
        const int w = b % p.n_windows;
        // a window whose mask is known to be all zero needs no mask reads
        const bool mask_on = p.mask && (!p.mask_live || p.mask_live[w] != 0);
        float add[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            ok[j] = own_ok && o0 + 8 * g + j < NX;
            add[j] = 0.f;
        }
        if (OWNER_IS_KEY) {
#pragma unroll
            for (int j = 0; j < 8; j++) add[j] = s_add[(8 * g + j) * AS + 16 * wave + l16];
        } else if (p.side_vec) {
            // the 8 keys of this lane are consecutive entries of one bias / mask row; n % 8 == 0, so they
            // exist together or not at all
            if (ok[0]) {
                const int64_t ro = (int64_t)own * p.bias_sn + o0 + 8 * g;
                if (p.bias) {
                    const V8 bv = ld8<V8>(reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + ro);
#pragma unroll
                    for (int j = 0; j < 8; j++) add[j] += (float)bv[j];
                }
                if (mask_on) {
                    const int64_t mo = w * p.mask_sw + (int64_t)own * p.mask_sn + o0 + 8 * g;
                    if (p.mask_f32) {
                        const f32x4 m0 = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mo);
                        const f32x4 m1 = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mo + 4);
#pragma unroll
                        for (int j = 0; j < 4; j++) { add[j] += m0[j]; add[4 + j] += m1[j]; }
                    } else {
                        const V8 mv = ld8<V8>(reinterpret_cast<const E*>(p.mask) + mo);
#pragma unroll
                        for (int j = 0; j < 8; j++) add[j] += (float)mv[j];
                    }
                }
            }
        } else {
            const int k0 = o0 + 8 * g;
            const E* bptr = reinterpret_cast<const E*>(p.bias) + h * p.bias_sh + (int64_t)own * p.bias_sn + k0;
            const int64_t mo = w * p.mask_sw + (int64_t)own * p.mask_sn + k0;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (ok[j]) {
                    if (p.bias) add[j] += (float)bptr[j];
                    if (mask_on)
                        add[j] += p.mask_f32 ? reinterpret_cast<const float*>(p.mask)[mo + j]
                                             : (float)reinterpret_cast<const E*>(p.mask)[mo + j];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            z2[j] = sa[j >> 2][j & 3] * scale2 + (OWNER_IS_KEY ? add[j] : add[j] * kLog2e);
            dpv[j] = da[j >> 2][j & 3];
        }
    };
    // A operand = transpose of the staged tile, slab c, half dt: rows d = 32 c + 8 (m / 4) + 4 dt + m % 4,
    // so that this lane's accumulators hold d = 32 c + 8 g + 4 dt + i of its owner row
    auto tr0 = [&](int c, int dt) __attribute__((always_inline)) -> SV8 {
        const SE* lo = t0 + (8 * g + (l16 >> 2)) * S + 32 * c + 8 * (l16 & 3) + 4 * dt;
        return lds_tr8<kScoreDT>(lo, lo + 4 * S);
    };
    auto tr1 = [&](int c, int dt) __attribute__((always_inline)) -> V8 {
        const E* lo = t1 + (8 * g + (l16 >> 2)) * S + 32 * c + 8 * (l16 & 3) + 4 * dt;
        return lds_tr8<DT>(lo, lo + 4 * S);
    };

    f32x4 acc0[KS][2], acc1[KS][2];     // FWD: o; DQ: dq^; DKV: dk^ and dv
#pragma unroll
    for (int c = 0; c < KS; c++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int i = 0; i < 4; i++) { acc0[c][dt][i] = 0.f; acc1[c][dt][i] = 0.f; }

    if (MODE == G_DBIAS) {
        float db[8];
#pragma unroll
        for (int j = 0; j < 8; j++) db[j] = 0.f;
        Staged st;
        if (b0 < p.bw) fetch(b0, 32 * kb, st);
        for (int b = b0; b < p.bw; b += p.groups) {
            load_owner(b);
            __syncthreads();
            commit(st);
            __syncthreads();
            if (b + p.groups < p.bw) fetch(b + p.groups, 32 * kb, st);
            float z2[8], dpv[8];
            bool ok[8];
            tile(b, 32 * kb, z2, dpv, ok);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float pr = ok[j] ? fast_exp2(z2[j] - own_lse2) : 0.f;
                if (!(pr == pr)) pr = 0.f;     // a fully masked row: z2 = lse = -inf
                db[j] += pr * (dpv[j] - own_delta);
            }
        }
        if (own_ok) {
            float* dst = p.part_dbias + (((int64_t)grp * p.heads + h) * NQ + own) * NKEY;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int kj = 32 * kb + 8 * g + j;
                if (kj < NKEY) dst[kj] = db[j];
            }
        }
        return;
    }

    // dq = (dq^ - q^ (q^ . dq^)) / ||q||, dq^ = s * acc (the same for dk with k); dv = acc1
    auto finish_grad = [&](int b) __attribute__((always_inline)) {
        const T4& ts = OWNER_IS_KEY ? p.k : p.q;
        const T4& td = OWNER_IS_KEY ? p.dk : p.dq;
        float xh[KS][2][4];
        float proj = 0.f;
#pragma unroll
        for (int c = 0; c < KS; c++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                const int col = 32 * c + 8 * g + 4 * dt;
                V4 xv;
#pragma unroll
                for (int i = 0; i < 4; i++) xv[i] = (E)0.f;
                if (own_ok && col < d) xv = *reinterpret_cast<const V4*>(rowp(ts, b, own) + col);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    xh[c][dt][i] = (float)xv[i] * own_inv;
                    acc0[c][dt][i] *= scale_nat;
                    proj += xh[c][dt][i] * acc0[c][dt][i];
                }
            }
        proj = col_add(proj);
        if (own_ok) {
            E* drow = const_cast<E*>(rowp(td, b, own));
            E* vrow = const_cast<E*>(rowp(p.dv, b, own));
#pragma unroll
            for (int c = 0; c < KS; c++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
                    const int col = 32 * c + 8 * g + 4 * dt;
                    if (col < d) {
                        V4 ov, vv;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            ov[i] = (E)((acc0[c][dt][i] - xh[c][dt][i] * proj) * own_inv);
                            vv[i] = (E)acc1[c][dt][i];
                        }
                        *reinterpret_cast<V4*>(drow + col) = ov;
                        if (MODE == G_DKV) *reinterpret_cast<V4*>(vrow + col) = vv;
                    }
                }
            if (MODE == G_DQ && g == 0) p.dscale_rows[((int64_t)b * p.heads + h) * p.row_pad + own] = proj;
        }
    };

    float m_run = -INFINITY, l_run = 0.f;
    // one step of 32 other rows; dbr: this lane's 8 dbias sums of the step (WITH_DB) or nullptr
    Staged st;
    auto step = [&](int b, int o0, float* dbr) __attribute__((always_inline)) {
        if (o0 == 0) fetch(b, 0, st);      // first step of a unit; later ones were fetched a step ahead
        __syncthreads();
        commit(st);
        __syncthreads();
        if (o0 + 32 < NX) fetch(b, o0 + 32, st);
        float z2[8], dpv[8];
        bool ok[8];
        tile(b, o0, z2, dpv, ok);
        if (MODE == G_FWD) {
            float mloc = -INFINITY;
#pragma unroll
            for (int j = 0; j < 8; j++) mloc = fmaxf(mloc, ok[j] ? z2[j] : -INFINITY);
            const float mnew = fmaxf(m_run, col_max(mloc));
            const float msafe = mnew == -INFINITY ? 0.f : mnew;
            const float alpha = fast_exp2(m_run - msafe);
            V8 pb;
            float ls = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float pr = ok[j] ? fast_exp2(z2[j] - msafe) : 0.f;
                ls += pr;
                pb[j] = (E)pr;
            }
            l_run = l_run * alpha + ls;
            m_run = mnew;
#pragma unroll
            for (int c = 0; c < KS; c++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
#pragma unroll
                    for (int i = 0; i < 4; i++) acc0[c][dt][i] *= alpha;
                    acc0[c][dt] = Elem<DT>::mfma16(tr1(c, dt), pb, acc0[c][dt]);
                }
        } else {
            V8 pb;
            SV8 zb;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float l2 = OWNER_IS_KEY ? s_lse2[8 * g + j] : own_lse2;
                const float dl = OWNER_IS_KEY ? s_delta[8 * g + j] : own_delta;
                float pr = ok[j] ? fast_exp2(z2[j] - l2) : 0.f;
                if (!(pr == pr)) pr = 0.f;     // a fully masked row: z2 = lse = -inf
                pb[j] = (E)pr;
                const float dz = pr * (dpv[j] - dl);
                zb[j] = (SE)dz;
                if (WITH_DB) dbr[j] += dz;
            }
#pragma unroll
            for (int c = 0; c < KS; c++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
                    acc0[c][dt] = Elem<kScoreDT>::mfma16(tr0(c, dt), zb, acc0[c][dt]);
                    if (MODE == G_DKV) acc1[c][dt] = Elem<DT>::mfma16(tr1(c, dt), pb, acc1[c][dt]);
                }
        }
    };

    if (WITH_DB) {
        float db[8][8];
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
            for (int j = 0; j < 8; j++) db[t][j] = 0.f;
        for (int b = b0; b < p.bw; b += p.groups) {
            load_owner(b);
#pragma unroll
            for (int c = 0; c < KS; c++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc0[c][dt][i] = 0.f;
#pragma unroll
            for (int t = 0; t < 8; t++)
                if (32 * t < NX) step(b, 32 * t, db[t]);
            finish_grad(b);
        }
        if (own_ok) {
            float* dst = p.part_dbias + (((int64_t)grp * p.heads + h) * NQ + own) * NKEY;
#pragma unroll
            for (int t = 0; t < 8; t++)
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int kj = 32 * t + 8 * g + j;
                    if (kj < NKEY) dst[kj] = db[t][j];
                }
        }
        return;
    }

    const int b = b0;
    load_owner(b);
    for (int o0 = 0; o0 < NX; o0 += 32) step(b, o0, nullptr);

    // ---- epilogue: this lane holds columns 32 c + 8 g + 4 dt + i of its owner row ----
    if (MODE == G_FWD) {
        const float l_tot = col_add(l_run);
        const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        if (own_ok) {
            E* orow = const_cast<E*>(rowp(p.o, b, own));
#pragma unroll
            for (int c = 0; c < KS; c++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
                    const int col = 32 * c + 8 * g + 4 * dt;
                    if (col < d) {
                        V4 ov;
#pragma unroll
                        for (int i = 0; i < 4; i++) ov[i] = (E)(acc0[c][dt][i] * inv_l);
                        *reinterpret_cast<V4*>(orow + col) = ov;
                    }
                }
            if (g == 0)
                p.lse[b * p.lse_sb + h * p.lse_sh + own] = l_tot > 0.f ? (m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
        }
        return;
    }

    if (MODE != G_FWD) finish_grad(b);
}

// dbias[h, q, k] = sum over the groups' partial tiles in a fixed order: 32 elements per workgroup, the
// groups dealt to 8 slices that are combined at the end.
template <int DT>
__global__ void __launch_bounds__(256) generic_dbias_reduce(const GenParams p) {
    typedef typename Elem<DT>::E E;
    __shared__ float part[8][32];
    const int64_t per = (int64_t)p.heads * p.n * p.nk;
    const int e = threadIdx.x & 31, sl = threadIdx.x >> 5;
    const int64_t i = (int64_t)blockIdx.x * 32 + e;
    float s = 0.f;
    if (i < per)
        for (int g = sl; g < p.groups; g += 8) s += p.part_dbias[g * per + i];
    part[sl][e] = s;
    __syncthreads();
    if (sl == 0 && i < per) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) t += part[k][e];
        reinterpret_cast<E*>(p.dbias)[i] = (E)t;
    }
}

// dlogit_scale[h] = [l <= ln 100] * sum over every query row of the head, in a fixed order: kDsSlices
// workgroups per head sum the units b = slice, slice + kDsSlices, ... into one partial each (kept in the
// delta buffer, which nobody reads any more), a last small kernel adds the partials.
constexpr int kDsSlices = 128;
__global__ void __launch_bounds__(256) generic_dscale_partial(const GenParams p) {
    __shared__ float part[256];
    const int h = blockIdx.x / kDsSlices, sl = blockIdx.x % kDsSlices;
    float s = 0.f;
    for (int b = sl; b < p.bw; b += kDsSlices) {
        const float* row = p.dscale_rows + ((int64_t)b * p.heads + h) * p.row_pad;
        for (int q = threadIdx.x; q < p.n; q += 256) s += row[q];
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off) part[threadIdx.x] += part[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) p.delta[blockIdx.x] = part[0];
}
template <int DT>
__global__ void __launch_bounds__(64) generic_dscale_final(const GenParams p) {
    typedef typename Elem<DT>::E E;
    const int h = blockIdx.x;
    if (threadIdx.x != 0) return;
    float s = 0.f;
    for (int k = 0; k < kDsSlices; k++) s += p.delta[h * kDsSlices + k];
    const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
    reinterpret_cast<E*>(p.dscale)[h] = (E)(ls <= kLn100 ? s : 0.f);
}

// ---- host side -----------------------------------------------------------------
static size_t align256g(size_t x) { return (x + 255) & ~(size_t)255; }

constexpr int kDbInDqMaxN = 256;   // windows up to this size sum dbias inside the dq pass

// Unit groups of the pass that sums dbias: enough workgroups to fill the chip, bounded partial tiles.
static int generic_groups(int heads, int n, int nk, int bw) {
    const int64_t chunks = (n + 63) / 64, kblocks = (nk + 31) / 32;
    int64_t groups;
    if (nk <= kDbInDqMaxN) {
        groups = 1024 / (heads * chunks);
        const int64_t cap = ((int64_t)64 << 20) / ((int64_t)heads * n * nk * 4);
        if (groups > cap) groups = cap;
    } else {
        groups = 2048 / (heads * chunks * kblocks);
        if (groups > 64) groups = 64;
    }
    if (groups < 1) groups = 1;
    if (groups > bw) groups = bw;
    return (int)groups;
}

// The tuned kernels cover head_dim 32 with as many keys as queries; everything else runs here.
bool generic_problem(int d, int n, int nk) { return d != 32 || nk != n; }

// One [BW * H, row_pad] fp32 buffer (delta, dscale rows); never smaller than the dscale partial sums.
static size_t generic_rows_bytes(int heads, int bw, size_t row_pad) {
    size_t rows = (size_t)bw * heads * row_pad;
    if (rows < (size_t)heads * kDsSlices) rows = (size_t)heads * kDsSlices;
    return align256g(rows * sizeof(float));
}

size_t generic_workspace_bytes(int heads, int n, int nk, int bw, bool has_bias) {
    const size_t row_pad = (size_t)((n + 63) / 64) * 64;
    size_t total = 2 * generic_rows_bytes(heads, bw, row_pad);
    if (has_bias) total += align256g((size_t)generic_groups(heads, n, nk, bw) * heads * n * nk * sizeof(float));
    return total;
}

template <int DT, int D>
static hipError_t launch_generic_d(const GenParams& p, bool backward, hipStream_t st) {
    const int chunks = (p.n + 63) / 64, kchunks = (p.nk + 63) / 64, kblocks = (p.nk + 31) / 32;
    const dim3 grid((unsigned)((int64_t)p.bw * p.heads * chunks)), gridk((unsigned)((int64_t)p.bw * p.heads * kchunks)), block(256);
    if (!backward) {
        hipLaunchKernelGGL((generic_kernel<DT, D, G_FWD>), grid, block, 0, st, p);
        return hipGetLastError();
    }
    const bool db_in_dq = p.bias && p.nk <= kDbInDqMaxN;
    if (db_in_dq) {
        const dim3 gq((unsigned)((int64_t)p.groups * p.heads * chunks));
        hipLaunchKernelGGL((generic_kernel<DT, D, G_DQ, true>), gq, block, 0, st, p);
    } else {
        hipLaunchKernelGGL((generic_kernel<DT, D, G_DQ>), grid, block, 0, st, p);
    }
    hipLaunchKernelGGL((generic_kernel<DT, D, G_DKV>), gridk, block, 0, st, p);
    if (p.bias) {
        if (!db_in_dq) {
            const dim3 gb((unsigned)((int64_t)p.groups * p.heads * chunks * kblocks));
            hipLaunchKernelGGL((generic_kernel<DT, D, G_DBIAS>), gb, block, 0, st, p);
        }
        const int64_t per = (int64_t)p.heads * p.n * p.nk;
        hipLaunchKernelGGL(generic_dbias_reduce<DT>, dim3((unsigned)((per + 31) / 32)), block, 0, st, p);
    }
    if (p.scale_kind == FWA2_SCALE_TENSOR && p.dscale) {
        // after DKV and DBIAS (same stream), so the delta buffer is free for the partial sums
        hipLaunchKernelGGL(generic_dscale_partial, dim3(p.heads * kDsSlices), block, 0, st, p);
        hipLaunchKernelGGL(generic_dscale_final<DT>, dim3(p.heads), dim3(64), 0, st, p);
    }
    return hipGetLastError();
}

template <int DT>
static hipError_t launch_generic_dt(const GenParams& p, bool backward, hipStream_t st) {
    if (p.d <= 32) return launch_generic_d<DT, 32>(p, backward, st);
    if (p.d <= 64) return launch_generic_d<DT, 64>(p, backward, st);
    return launch_generic_d<DT, 128>(p, backward, st);
}

// p: the caller's problem, already validated.  workspace (backward only): generic_workspace_bytes().
hipError_t launch_generic(const fwa2_problem* pr, bool backward) {
    GenParams p;
    memset(&p, 0, sizeof(p));
    auto t4 = [](const fwa2_tensor4& t) { return T4{t.ptr, t.stride_bw, t.stride_h, t.stride_n}; };
    p.q = t4(pr->q); p.k = t4(pr->k); p.v = t4(pr->v); p.o = t4(pr->o);
    p.d_o = t4(pr->d_o); p.dq = t4(pr->dq); p.dk = t4(pr->dk); p.dv = t4(pr->dv);
    if (pr->grid_h > 0) {
        p.map.nwx = pr->grid_w / pr->win_w;
        p.map.nw = (pr->grid_h / pr->win_h) * p.map.nwx;
        p.map.gh = pr->grid_h; p.map.gw = pr->grid_w;
        p.map.wh = pr->win_h; p.map.ww = pr->win_w;
        p.map.sh = pr->shift_h; p.map.sw = pr->shift_w;
        p.map.inv_ww = 65536 / pr->win_w + 1;
    }
    p.logit_scale = pr->logit_scale;
    p.scale_kind = pr->scale_kind;
    p.default_scale = 1.0f / sqrtf((float)(pr->scale_head_dim > 0 ? pr->scale_head_dim : pr->head_dim));
    p.bias = pr->bias.ptr; p.bias_sh = pr->bias.stride_a; p.bias_sn = pr->bias.stride_n;
    p.mask = pr->mask.ptr; p.mask_sw = pr->mask.stride_a; p.mask_sn = pr->mask.stride_n;
    p.mask_f32 = pr->mask.ptr && pr->mask_dtype == FWA2_F32;
    p.n_windows = pr->mask.ptr ? pr->n_windows : 1;
    p.mask_live = pr->mask.ptr ? pr->mask_live : nullptr;
    auto rows16 = [&](const fwa2_tensor3& t, int esize) {
        return t.ptr == nullptr || (((uintptr_t)t.ptr & 15) == 0 && (t.stride_a * esize) % 16 == 0 && (t.stride_n * esize) % 16 == 0);
    };
    p.side_vec = (pr->n_keys > 0 ? pr->n_keys : pr->n) % 8 == 0 && rows16(pr->bias, 2) && rows16(pr->mask, pr->mask_dtype == FWA2_F32 ? 4 : 2);
    p.lse = pr->lse; p.lse_sb = pr->lse_stride_bw; p.lse_sh = pr->lse_stride_h;
    p.bw = pr->bw; p.heads = pr->heads; p.n = pr->n; p.d = pr->head_dim;
    p.nk = pr->n_keys > 0 ? pr->n_keys : pr->n;
    p.row_pad = ((pr->n + 63) / 64) * 64;
    if (backward) {
        unsigned char* ws = reinterpret_cast<unsigned char*>(pr->workspace);
        const size_t rows = generic_rows_bytes(p.heads, p.bw, (size_t)p.row_pad);
        p.delta = reinterpret_cast<float*>(ws);
        p.dscale_rows = reinterpret_cast<float*>(ws + rows);
        p.part_dbias = reinterpret_cast<float*>(ws + 2 * rows);
        p.groups = generic_groups(p.heads, p.n, p.nk, p.bw);
        p.dbias = pr->dbias;
        p.dscale = pr->dscale;
    }
    hipStream_t st = (hipStream_t)pr->stream;
    if (pr->dtype == FWA2_BF16) return launch_generic_dt<FWA2_BF16>(p, backward, st);
    return launch_generic_dt<FWA2_F16>(p, backward, st);
}

}  // namespace fwa2
