// Backward, key side: dk, dv and dbias for gfx950 (dq lives in fwa2_bwd_dq.hip).
//
// Replaces _bwd_preprocess_do_o_dot, the dK/dV/dbias half of _bwd_kernel and
// the host epilogue of the reference
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:6-51, 84-564, 703-711).
//
// Work split.  A workgroup is PERSISTENT for one head: it walks over many
// (batch*window) units of that head and keeps the bias-gradient tile in
// registers for the whole walk, so dbias costs one register add per score and
// one plain store per workgroup instead of one global atomic per score
// (attn_kernel_backward.py:273).  Inside a workgroup every wavefront owns 16 or
// 32 keys and streams all queries of the unit past them, 32 at a time; the
// wavefronts only meet at the two barriers around the per-unit load.
//
// Per unit:
//   load     q (L2-normalised, times s*log2e) and dO -> LDS in the input dtype;
//            k_hat -> LDS (each wavefront then takes its own rows as an MFMA
//            operand); -delta = -rowsum(o*dO) and -lse*log2e -> LDS.
//   blocks   S = Q_hat K_hat^T and dP = dO V^T with v_mfma_f32_16x16x32 (rows =
//            queries, columns = this wave's keys; -lse and -delta ride in as the
//            accumulator inits), P = 2^(S+bias+mask-lse), dZ = P (dP - delta);
//            dbias registers += dZ; the accumulators, rounded to the input dtype,
//            are directly the B operands (k = queries) of dV^T += dO^T P and
//            dK_hat^T += Q_hat^T dZ, whose A operands come out of the row-major
//            LDS tiles with ds_read_b64_tr_b16.
//   epilogue dk = (dk_hat - k_hat (dk_hat.k_hat)) / |k| in registers, dv as is.
//
// bias and mask are read key-major (transposed once per call by a small
// pre-pass into the workspace) so that a lane's scores are one vector load,
// and are fetched one block ahead of their use.
#include <atomic>

#include "fwa2_common.hpp"

// FWA2_HALF splits this translation unit for the build: 0 (default) the whole file; 1 everything except the
// fp16 instantiations, which it reaches through launch_backward_f16(); 2 the fp16 instantiations alone.
#ifndef FWA2_HALF
#define FWA2_HALF 0
#endif

namespace fwa2 {

constexpr int kRow = 40;    // LDS row stride of 16-bit tiles, in elements (80 bytes)


// Per-wavefront state that lives in registers across the query blocks of one unit (dvacc,
// dkacc, bk, bv) or across all units of the workgroup (dbacc).
template <int DT, int NQB, int KT>
struct WaveRegs {
    float dbacc[NQB][KT][8];
    f32x4 dvacc[KT][2], dkacc[KT][2];
    typename Elem<kScoreDT>::V8 bk[KT];
    typename Elem<DT>::V8 bv[KT];
};

// LDS views of one workgroup.  The arrays behind them are separate __shared__ variables with
// compile-time sizes: tile addresses are lane offset + immediate, and the compiler can tell the
// landing area (written by global_load_lds) from the tiles, so reads of the tiles do not wait
// for fetches in flight.
template <int DT, int NQB>
struct BwdLds {
    typedef typename Elem<DT>::E E;
    static constexpr int R = 32 * NQB;
    // q_hat and k_hat are kept in the score type of the forward kernel (fp16 also for bf16 inputs), so that the
    // recomputed scores round as the forward's did and P sums to 1 against the forward's lse
    typename Elem<kScoreDT>::E* Qs;   // q_hat * s * log2e, row-major [query][kRow]
    typename Elem<kScoreDT>::E* Ks;   // k_hat, [key][kRow]
    E* dOs;         // dO, [query][kRow]
    float* nlse2;   // -lse * log2e   (-inf for padded / fully masked rows)
    float* ndelta;  // -rowsum(o * dO)
    float* kinv;    // 1 / max(|k|, eps), negated when |k| <= eps
    // landing area of the next unit's rows: unpadded 64-byte rows, rows >= n stay zero
    E *rawQ, *rawK, *rawV, *rawDO, *rawO;
    float* rawLse;
};

// 16 bytes per lane straight from global memory into LDS (no registers held while in flight):
// lane i of the wavefront lands at lds_wave_base + 16 i.
template <class E>
__device__ __forceinline__ void async_row_chunk(const E* gsrc, E* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, kStreamPolicy);
}

// All query blocks of one unit.  MASKED is uniform per unit (the window's mask is live or not),
// so the whole block sequence exists twice instead of branching inside every block.
// `block_start(qb)` runs at the top of every block, after every side value fetched for that block
// has arrived (the kernel uses it to start the next unit's fetch behind them).
template <int DT, bool HAS_BIAS, class ME, int NQB, int KT, bool MASKED, bool BIG, class Hook>
__device__ __forceinline__ void unit_blocks(BwdLds<DT, NQB>& L, WaveRegs<DT, NQB, KT>& w,
                                            const typename Elem<DT>::E* bias_t, const ME* mask_t, int n, int nqb,
                                            int l16, int g, int key0, bool tail_keys, int side_stride_big,
                                            Hook block_start) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    typedef ME MV4 __attribute__((ext_vector_type(4)));
    constexpr int R = 32 * NQB;
    const int SS = BIG ? side_stride_big : R;    // row stride of the key-major side tables

    // bias (and mask) values of the coming block travel in registers: they are fetched one block
    // ahead so that the L2 round trip overlaps the rest of the block instead of stalling it
    V4 bcur[KT][2];
    MV4 mcur[KT][2];
    auto fetch_side = [&](int qbn) __attribute__((always_inline)) {
        const int q8n = 32 * qbn + 8 * g;
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
                if (HAS_BIAS) bcur[kt][t] = *reinterpret_cast<const V4*>(bias_t + (int64_t)16 * kt * SS + q8n + 4 * t);
                if (MASKED) mcur[kt][t] = *reinterpret_cast<const MV4*>(mask_t + (int64_t)16 * kt * SS + q8n + 4 * t);
            }
    };
    fetch_side(0);

    // The operands of a block's first query tile (q_hat and dO rows, -lse and -delta) are read from LDS while the
    // previous block finishes, so that a block does not open with a wait for them.
    // (with a live mask only the two rows: the mask values in flight take the registers of the accumulator inits;
    // not with one key tile per wavefront, where the budget is 128 registers and any of it would spill)
    constexpr bool PF = KT == 2;              // the two rows
    constexpr bool PFI = !MASKED && KT == 2;  // and the accumulator inits
    SV8 aq0;
    V8 ado0;
    f32x4 nl0, nd0;
    auto fetch_first = [&](int qbn) __attribute__((always_inline)) {
        if (!PF) return;
        const int rowq = 32 * qbn + 8 * (l16 >> 2) + (l16 & 3);
        aq0 = ld8<SV8>(L.Qs + rowq * kRow + 8 * g);
        ado0 = ld8<V8>(L.dOs + rowq * kRow + 8 * g);
        if (PFI) {
            nl0 = *reinterpret_cast<const f32x4*>(L.nlse2 + 32 * qbn + 8 * g);
            nd0 = *reinterpret_cast<const f32x4*>(L.ndelta + 32 * qbn + 8 * g);
        }
    };
    fetch_first(0);

#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        if (qb < nqb) {
            const int q8 = 32 * qb + 8 * g;          // first of this lane's 8 queries
            // every side value of this block is waited for here, in one go ...
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    if (HAS_BIAS) asm volatile("" : "+v"(bcur[kt][t]));
                    if (MASKED) asm volatile("" : "+v"(mcur[kt][t]));
                }
            block_start(qb);   // ... so that whatever this issues is younger than all of them
            // ---- phase A, one key tile at a time ----
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
                V8 p8;
                SV8 z8;     // dZ in the score type: its partner in the dK product is q_hat
                // k_hat of the lane's key is re-read per block: 4 registers less per key tile than keeping it
                const SV8 bk_now = ld8<SV8>(L.Ks + (key0 + 16 * kt) * kRow + 8 * g);
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const int rowq = 32 * qb + 8 * (l16 >> 2) + 4 * t + (l16 & 3);
                    const SV8 aq = (PF && t == 0) ? aq0 : ld8<SV8>(L.Qs + rowq * kRow + 8 * g);
                    const V8 ado = (PF && t == 0) ? ado0 : ld8<V8>(L.dOs + rowq * kRow + 8 * g);
                    // accumulator inits: -lse*log2e and -delta of this lane's 4 queries
                    const f32x4 nl = (PFI && t == 0) ? nl0 : *reinterpret_cast<const f32x4*>(L.nlse2 + q8 + 4 * t);
                    const f32x4 nd = (PFI && t == 0) ? nd0 : *reinterpret_cast<const f32x4*>(L.ndelta + q8 + 4 * t);
                    f32x4 sacc = Elem<kScoreDT>::mfma16(aq, bk_now, nl);      // (S - lse) * log2e
                    const f32x4 pacc = Elem<DT>::mfma16(ado, w.bv[kt], nd);   // dP - delta
                    if (HAS_BIAS) {   // padded key rows of bias_t hold -inf
#pragma unroll
                        for (int i = 0; i < 4; i++) sacc[i] = fmaf((float)bcur[kt][t][i], kLog2e, sacc[i]);
                    }
                    if (MASKED) {
#pragma unroll
                        for (int i = 0; i < 4; i++) sacc[i] = fmaf((float)mcur[kt][t][i], kLog2e, sacc[i]);
                    }
                    if (!HAS_BIAS) {
                        if (tail_keys) {
#pragma unroll
                            for (int i = 0; i < 4; i++) sacc[i] = (key0 + 16 * kt < n) ? sacc[i] : -INFINITY;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float pj = fast_exp2(sacc[i]);
                        const float dz = pj * pacc[i];
                        if (HAS_BIAS) w.dbacc[qb][kt][4 * t + i] += dz;
                        p8[4 * t + i] = (E)pj;
                        z8[4 * t + i] = (SE)dz;
                    }
                }
                if (kt == KT - 1 && qb + 1 < NQB) fetch_first(qb + 1);   // the first tile's operands are dead by now
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
                    // A row m <-> d = 8 (m / 4) + 4 dt + m % 4: the lane's dk / dv values are d = 8g + 4dt + i
                    const int off = (q8 + (l16 >> 2)) * kRow + 8 * (l16 & 3) + 4 * dt;
                    const V8 a_do = lds_tr8<DT>(L.dOs + off, L.dOs + off + 4 * kRow);
                    w.dvacc[kt][dt] = Elem<DT>::mfma16(a_do, p8, w.dvacc[kt][dt]);
                    const SV8 a_q = lds_tr8<kScoreDT>(L.Qs + off, L.Qs + off + 4 * kRow);
                    w.dkacc[kt][dt] = Elem<kScoreDT>::mfma16(a_q, z8, w.dkacc[kt][dt]);
                }
            }
            fetch_side(qb + 1 < nqb ? qb + 1 : 0);
        }
    }
}

// KT = key tiles of 16 owned by one wavefront, NQB = compile-time bound on query blocks of 32.
// Units whose window mask is live run the MASKED copy of the block sequence, the others the plain
// one (uniform per unit, so no block ever branches on the mask).  MODE 2: one launch walks both
// kinds (windows of up to 128 tokens, where both copies fit the register file without scratch);
// MODE 0 / 1: a launch for the units with an all-zero mask and one for the others.
// BIG: windows of more than 256 tokens.  The N x N score matrix is cut into 256 x 256 (or 192 x 192) super-tiles;
// a workgroup then belongs to one (head, query chunk, key chunk), reads only those rows, keeps that
// tile of dbias in registers and writes its share of dk / dv (already taken back through the
// normalisation, which is linear) as fp32 partials that are summed over the query chunks by workgroups of the dq launch (dkv_reduce_rows).
// MAPPED: rows are addressed through the window map (cyclic shift + window partition done here).  BIG decides that
// at run time (p.map.nw > 0): its row fetches are a small part of a super-tile's work.
template <int DT, bool HAS_BIAS, int MASK_DT, int NQB, int KT, int MODE, bool BIG, bool MAPPED = false>
__global__ void __launch_bounds__(NQB * 128 / KT) bwd_kernel(const BwdParams p) {
    static_assert(!(MAPPED && BIG), "with BIG the map is a run-time property (p.map.nw > 0)");
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename MaskElem<DT, MASK_DT>::E ME;

    constexpr int R = 32 * NQB;            // padded rows of every LDS tile (and of the side tables unless BIG)
    const int NPk = p.waves * 16 * KT;     // padded key rows of this workgroup
    // ---- which head (and, for BIG, which super-tile) this workgroup owns ----
    int h, grp, q_off = 0, k_off = 0, qs = 0;
    if (BIG) {
        // Workgroups go to the 8 XCDs in turn, each with an L2 of its own.  The super-tiles of one (head, group) --
        // workgroups that walk the same units at the same pace -- are given to workgroups 8 apart, so one XCD fetches
        // a unit's rows once for all of them.
        // (Only when the (head, group) pairs divide evenly among the XCDs: otherwise some XCDs would hold one pair's
        // workgroups more than others, which costs more than the shared fetches save -- +2 % at 1024 tokens, where
        // 12 pairs of 16 super-tiles would fill four XCDs and half-fill the other four.)
        const int tiles = p.n_chunks * p.n_chunks;
        int tile, sid;
        if (p.big_xcd) {
            const int pos = blockIdx.x >> 3;
            tile = pos % tiles;
            sid = (pos / tiles) * 8 + (blockIdx.x & 7);
        } else {
            tile = (blockIdx.x / p.groups) % tiles;
            sid = (blockIdx.x / (p.groups * tiles)) * p.groups + blockIdx.x % p.groups;
        }
        h = sid / p.groups;
        grp = sid - h * p.groups;
        qs = tile / p.n_chunks;
        const int ks = tile - qs * p.n_chunks;
        q_off = qs * R;
        k_off = ks * NPk;
    } else {
        h = blockIdx.x / p.groups;
        grp = blockIdx.x - h * p.groups;
    }
    const int N = BIG ? min(p.n - q_off, R) : p.n;        // query rows of this workgroup
    const int NK = BIG ? min(p.n - k_off, NPk) : p.n;     // key rows of this workgroup
    const int R_tot = BIG ? p.r_tot : R;                  // row stride / padded keys of the side tables
    const int NPk_tot = BIG ? p.npk_tot : NPk;
    const int nqb = (N + 31) >> 5;         // query blocks of 32 that hold real rows

    typedef typename Elem<kScoreDT>::E SE;
    typedef typename Elem<kScoreDT>::V8 SV8;
    typedef typename Elem<kScoreDT>::V4 SV4;
    __shared__ __attribute__((aligned(16))) SE lds_Qs[R * kRow];
    __shared__ __attribute__((aligned(16))) SE lds_Ks[R * kRow];
    __shared__ __attribute__((aligned(16))) E lds_dOs[R * kRow];
    __shared__ __attribute__((aligned(16))) float lds_nlse2[R];
    __shared__ __attribute__((aligned(16))) float lds_ndelta[R];
    __shared__ __attribute__((aligned(16))) float lds_kinv[R];
    __shared__ __attribute__((aligned(16))) E lds_rawQ[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawK[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawV[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawDO[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawO[R * 32];
    __shared__ __attribute__((aligned(16))) float lds_rawLse[R];
    BwdLds<DT, NQB> L;
    L.Qs = lds_Qs; L.Ks = lds_Ks; L.dOs = lds_dOs; L.nlse2 = lds_nlse2; L.ndelta = lds_ndelta; L.kinv = lds_kinv;
    L.rawQ = lds_rawQ; L.rawK = lds_rawK; L.rawV = lds_rawV; L.rawDO = lds_rawDO; L.rawO = lds_rawO;
    L.rawLse = lds_rawLse;

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane_0 = tid & 63;
    const int wave_0 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = lane_0, wave = wave_0;

    float s_true;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        s_true = expf(fminf(ls, kLn100));
    } else {
        s_true = p.default_scale;
    }
    const float scale2 = s_true * kLog2e;

    const bool tail_keys = NPk > NK;        // some key columns are padding

    WaveRegs<DT, NQB, KT> w;
#pragma unroll
    for (int a = 0; a < NQB; a++)
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int j = 0; j < 8; j++) w.dbacc[a][kt][j] = 0.f;
    // key-major side tables: uniform base of this workgroup's keys; the lane's row is added per unit
    const E* bias_base = nullptr;
    if (HAS_BIAS) bias_base = reinterpret_cast<const E*>(p.bias_t) + ((int64_t)h * NPk_tot + k_off) * R_tot + q_off;

    // ---- the order in which the head's units are dealt out.  With the mask flags at hand the windows
    // are listed once, those with a live mask first: ranks t < t_live are the units of the live
    // windows, the rest those of the all-zero windows, each group image by image.  Every workgroup
    // walks t = grp, grp + groups, ..., so all get the same number of units (to within one) whatever
    // the pattern of masked windows, and the workgroups running at any moment read neighbouring
    // units.  Without the flags every unit of a masked call counts as live. ----
    __shared__ uint8_t lds_live[kLiveCache];
    __shared__ uint16_t lds_list[kLiveCache];
    __shared__ int lds_count;
    const bool listed = MASK_DT >= 0 && p.mask_live && p.n_windows <= kLiveCache;
    if (listed) {
        for (int i = tid; i < p.n_windows; i += nthreads) lds_live[i] = p.mask_live[i];
        __syncthreads();
        if (wave_0 == 0) {
            int cnt = 0;
#pragma unroll 1
            for (int cls = 1; cls >= 0; cls--) {
                for (int base = 0; base < p.n_windows; base += 64) {
                    const int w = base + lane_0;
                    const bool in = w < p.n_windows && ((lds_live[w] != 0) == (cls != 0));
                    const unsigned long long bal = __ballot(in);
                    if (in) lds_list[cnt + __popcll(bal & ((1ull << lane_0) - 1ull))] = (uint16_t)w;
                    cnt += __popcll(bal);
                }
                if (cls == 1 && lane_0 == 0) lds_count = cnt;
            }
        }
        __syncthreads();
    }
    const int n_live = listed ? __builtin_amdgcn_readfirstlane(lds_count) : 0;
    const int n_img = (p.bw + p.n_windows - 1) / p.n_windows;
    const int t_live = listed ? n_img * n_live : (MASK_DT >= 0 ? p.bw : 0);
    const int total = listed ? n_img * p.n_windows : p.bw;
    const int t_begin = MODE == 0 ? t_live : 0;              // ranks this launch deals out
    const int t_end = MODE == 1 ? t_live : total;
    auto unit_of = [&](int t) -> int {
        if (!listed) return t;
        int img, wi;
        if (t < t_live) {
            img = t / n_live;
            wi = t - img * n_live;
        } else {
            const int n_rest = p.n_windows - n_live;
            const int u = t - t_live;
            img = u / n_rest;
            wi = n_live + (u - img * n_rest);
        }
        return __builtin_amdgcn_readfirstlane(img * p.n_windows + (int)lds_list[wi]);
    };
    // first rank >= t (in steps of the group count) that names an existing unit
    auto rank_from = [&](int t) -> int {
        for (; t < t_end; t += p.groups)
            if (unit_of(t) < p.bw) return t;
        return t_end;
    };
    // ---- asynchronous fetch of one unit's rows into the landing area ----
    auto fetch_unit = [&](int b) __attribute__((always_inline)) {
        const E* qptr = reinterpret_cast<const E*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + q_off * p.q.sn;
        const E* kptr = reinterpret_cast<const E*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + k_off * p.k.sn;
        const E* vptr = reinterpret_cast<const E*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + k_off * p.v.sn;
        const E* optr = reinterpret_cast<const E*>(p.o.ptr) + b * p.o.sb + h * p.o.sh + q_off * p.o.sn;
        const E* doptr = reinterpret_cast<const E*>(p.d_o.ptr) + b * p.d_o.sb + h * p.d_o.sh + q_off * p.d_o.sn;
        const float* lseptr = p.lse + b * p.lse_sb + h * p.lse_sh + q_off;
        // re-materialised here so that no per-row address is computed ahead of time and spilled
        // (a spill reload would wait for every fetch already in flight)
        const int lane = lane_now();
        int wave = wave_0;
        asm volatile("" : "+s"(wave));
        const int dc = (lane & 3) * 8;
        for (int row0 = wave * 16; row0 < R; row0 += 16 * p.waves) {   // 16 rows per wavefront and instruction
            const int r = row0 + (lane >> 2);
            if constexpr (MAPPED) {
                if (r < N) {
                    const int pos = unit_row<true>(p.map, b, r);
                    async_row_chunk(row_at(unit_ptr<true, E>(p.q, p.map, b, h), pos, p.q.sn, dc), L.rawQ + row0 * 32);
                    async_row_chunk(row_at(unit_ptr<true, E>(p.d_o, p.map, b, h), pos, p.d_o.sn, dc), L.rawDO + row0 * 32);
                    async_row_chunk(row_at(unit_ptr<true, E>(p.o, p.map, b, h), pos, p.o.sn, dc), L.rawO + row0 * 32);
                    async_row_chunk(row_at(unit_ptr<true, E>(p.k, p.map, b, h), pos, p.k.sn, dc), L.rawK + row0 * 32);
                }
                continue;
            }
            if constexpr (BIG) {
                if (p.map.nw > 0) {
                    if (r < N) {
                        const int pos = unit_row<true>(p.map, b, q_off + r);
                        async_row_chunk(row_at(unit_ptr<true, E>(p.q, p.map, b, h), pos, p.q.sn, dc), L.rawQ + row0 * 32);
                        async_row_chunk(row_at(unit_ptr<true, E>(p.d_o, p.map, b, h), pos, p.d_o.sn, dc), L.rawDO + row0 * 32);
                        async_row_chunk(row_at(unit_ptr<true, E>(p.o, p.map, b, h), pos, p.o.sn, dc), L.rawO + row0 * 32);
                    }
                    if (r < NK)
                        async_row_chunk(row_ptr<true, E>(p.k, p.map, b, h, k_off + r, dc), L.rawK + row0 * 32);
                    continue;
                }
            }
            if (r < N) {
                async_row_chunk(row_at(qptr, r, p.q.sn, dc), L.rawQ + row0 * 32);
                async_row_chunk(row_at(doptr, r, p.d_o.sn, dc), L.rawDO + row0 * 32);
                async_row_chunk(row_at(optr, r, p.o.sn, dc), L.rawO + row0 * 32);
            }
            if (r < NK) async_row_chunk(row_at(kptr, r, p.k.sn, dc), L.rawK + row0 * 32);
        }
        // v: every wavefront fetches exactly the key rows it owns, so nobody else reads them
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int row0 = (wave * KT + kt) * 16;
            const int r = row0 + (lane >> 2);
            if constexpr (MAPPED) {
                if (r < NK) async_row_chunk(row_ptr<true, E>(p.v, p.map, b, h, r, dc), L.rawV + row0 * 32);
                continue;
            }
            if constexpr (BIG) {
                if (p.map.nw > 0) {
                    if (r < NK) async_row_chunk(row_ptr<true, E>(p.v, p.map, b, h, k_off + r, dc), L.rawV + row0 * 32);
                    continue;
                }
            }
            if (r < NK) async_row_chunk(row_at(vptr, r, p.v.sn, dc), L.rawV + row0 * 32);
        }
        for (int r0 = wave * 64; r0 < N; r0 += 64 * p.waves) {
            if (r0 + lane < N)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(lseptr + r0 + lane),
                                                 (__attribute__((address_space(3))) void*)(L.rawLse + r0), 4, 0, kStreamPolicy);
        }
    };

    // landing rows beyond n must read as zeros for the whole kernel
    for (int i = tid; i < R * 32 / 8; i += nthreads) {
        st8<V8>(L.rawQ + i * 8, zero8<V8>()); st8<V8>(L.rawK + i * 8, zero8<V8>()); st8<V8>(L.rawV + i * 8, zero8<V8>());
        st8<V8>(L.rawDO + i * 8, zero8<V8>()); st8<V8>(L.rawO + i * 8, zero8<V8>());
    }
    __syncthreads();

    int t = rank_from(t_begin + grp);
    if (t < t_end) fetch_unit(unit_of(t));

    while (t < t_end) {
        const int b = unit_of(t);
        const int t_next = rank_from(t + p.groups);
        const int b_next = t_next < t_end ? unit_of(t_next) : p.bw;
        const bool live = MODE != 0 && MASK_DT >= 0 && t < t_live;     // this unit's window mask has non-zero entries
        const ME* mask_base = nullptr;
        if (live) {
            const int wnd = b % p.n_windows;
            mask_base = reinterpret_cast<const ME*>(p.mask_t) + ((int64_t)wnd * NPk_tot + k_off) * R_tot + q_off;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's share of the unit has landed
        __syncthreads();   // ... and everybody's; the previous unit is done with the tiles
        // ---- landing area -> MFMA tiles: one 8-element chunk of a row per thread and pass ----
        {
            const int st = wave_0 * 64 + lane_now();
            const int dc = (st & 3) * 8;
            for (int r = st >> 2; r < R; r += nthreads >> 2) {
                float xq[8], xk[8], xd[8], xo[8];
                const V8 do8 = ld8<V8>(L.rawDO + r * 32 + dc);
                unpack8(ld8<V8>(L.rawQ + r * 32 + dc), xq);
                unpack8(ld8<V8>(L.rawK + r * 32 + dc), xk);
                unpack8(do8, xd);
                unpack8(ld8<V8>(L.rawO + r * 32 + dc), xo);
                float sq = 0.f, sk = 0.f, dl = 0.f;
#pragma unroll
                for (int j = 0; j < 8; j++) { sq += xq[j] * xq[j]; sk += xk[j] * xk[j]; dl += xo[j] * xd[j]; }
                sq = quad_add(sq); sk = quad_add(sk); dl = quad_add(dl);
                const float iq = inv_norm(sq) * scale2, ik = inv_norm(sk);
                SV8 qn, kn;
#pragma unroll
                for (int j = 0; j < 8; j++) { qn[j] = (SE)(xq[j] * iq); kn[j] = (SE)(xk[j] * ik); }
                st8<SV8>(L.Qs + r * kRow + dc, qn);
                st8<SV8>(L.Ks + r * kRow + dc, kn);
                st8<V8>(L.dOs + r * kRow + dc, do8);
                if ((st & 3) == 0) {
                    L.ndelta[r] = -dl;
                    if (!BIG && r < N) p.delta[((int64_t)b * p.heads + h) * p.delta_stride + r] = dl;   // for the dq kernel
                }
                if ((st & 3) == 1) {
                    float l2 = -INFINITY;          // padded / fully masked rows: P = 0
                    if (r < N) { const float l = L.rawLse[r]; l2 = (l == -INFINITY) ? -INFINITY : -l * kLog2e; }
                    L.nlse2[r] = l2;
                }
                if ((st & 3) == 2) L.kinv[r] = (sqrtf(sk) > kNormEps) ? ik : -ik;
            }
        }
        // lane-derived values of the blocks and the epilogue are made here, once per unit, so that
        // neither they nor the addresses built on them live (or sit in scratch) across units
        const int ln = lane_now();
        const int l16 = ln & 15, g = ln >> 4;
        const int key0 = wave_0 * 16 * KT + l16;        // this lane's key in key tile 0 (tile kt: + 16 kt)
        const E* bias_t = HAS_BIAS ? bias_base + key0 * R_tot : nullptr;
        const ME* mask_t = live ? mask_base + key0 * R_tot : nullptr;
#pragma unroll
        for (int kt = 0; kt < KT; kt++) w.bv[kt] = ld8<V8>(L.rawV + (key0 + 16 * kt) * 32 + 8 * g);
        __syncthreads();   // tiles complete; the landing area is free again
#pragma unroll
        for (int kt = 0; kt < KT; kt++) w.bk[kt] = ld8<SV8>(L.Ks + (key0 + 16 * kt) * kRow + 8 * g);
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
#pragma unroll
                for (int i = 0; i < 4; i++) { w.dvacc[kt][dt][i] = 0.f; w.dkacc[kt][dt][i] = 0.f; }

        // The next unit's fetch starts at the top of the last block: memory returns in issue order,
        // so an earlier start would make every later wait for bias values also wait for the fetch.
        const int fetch_at = nqb - 1;
        auto block_start = [&](int qb) __attribute__((always_inline)) {
            if (qb == fetch_at && b_next < p.bw) fetch_unit(b_next);
            // The SIMD favours its older wavefront, so the younger one of each pair would finish the
            // blocks long after it and run the tail alone; raising its priority after the first quarter
            // lets both reach the end of the unit together.
            if (qb == NQB / 4 && wave_0 >= (p.waves >> 1)) __builtin_amdgcn_s_setprio(2);
        };
        if (MODE == 1 || (MODE == 2 && live))
            unit_blocks<DT, HAS_BIAS, ME, NQB, KT, MASK_DT >= 0, BIG>(L, w, bias_t, mask_t, NK, nqb, l16, g, key0, tail_keys,
                                                                      R_tot, block_start);
        else
            unit_blocks<DT, HAS_BIAS, ME, NQB, KT, false, BIG>(L, w, bias_t, mask_t, NK, nqb, l16, g, key0, tail_keys, R_tot,
                                                               block_start);
        __builtin_amdgcn_s_setprio(0);

        // ---- epilogue dk, dv: lane (key, g) holds d = 8g + 4dt + i (16 bytes of a row); k_hat and 1/|k| come from LDS ----
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int key = key0 + 16 * kt;
            const bool key_ok = key < NK;
            float x[8], a[8];
            float dot = 0.f;
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                const SV4 k4 = *reinterpret_cast<const SV4*>(L.Ks + key * kRow + 8 * g + 4 * dt);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    x[4 * dt + i] = (float)k4[i];
                    a[4 * dt + i] = w.dkacc[kt][dt][i] * kLn2;      // undo the log2e folded into Q_hat
                    dot += a[4 * dt + i] * x[4 * dt + i];
                }
            }
            dot = xor32_add(xor16_add(dot));
            const float ki = L.kinv[key];
            const float inv = fabsf(ki);
            const float proj = ki > 0.f ? dot : 0.f;
            if (key_ok) {
                if (BIG) {
                    // fp32 partial of this query chunk: [qs][b][h][padded key][32]
                    const int64_t row = (((int64_t)qs * p.bw + b) * p.heads + h) * NPk_tot + k_off + key;
#pragma unroll
                    for (int dt = 0; dt < 2; dt++) {
                        f32x4 o4, v4;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            o4[i] = inv * (a[4 * dt + i] - x[4 * dt + i] * proj);
                            v4[i] = w.dvacc[kt][dt][i];
                        }
                        *reinterpret_cast<f32x4*>(p.part_dk + row * 32 + 8 * g + 4 * dt) = o4;
                        *reinterpret_cast<f32x4*>(p.part_dv + row * 32 + 8 * g + 4 * dt) = v4;
                    }
                } else {
                    E* dkp = const_cast<E*>(row_ptr<MAPPED, E>(p.dk, p.map, b, h, key));
                    E* dvp = const_cast<E*>(row_ptr<MAPPED, E>(p.dv, p.map, b, h, key));
                    V8 o8, v8;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        o8[j] = (E)(inv * (a[j] - x[j] * proj));
                        v8[j] = (E)w.dvacc[kt][j >> 2][j & 3];
                    }
                    st8_stream<V8>(dkp + 8 * g, o8);
                    st8_stream<V8>(dvp + 8 * g, v8);
                }
            }
        }
        t = t_next;
    }

    // ---- flush the per-workgroup partial sums ----
    if (HAS_BIAS) {
        const int ln = lane_now();
        const int g = ln >> 4;
        const int key0 = wave_0 * 16 * KT + (ln & 15);
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            float* dst = p.part_dbias + (((int64_t)h * p.db_parts + p.db_slot0 + grp) * NPk_tot + k_off + key0 + 16 * kt) * R_tot + q_off;
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) {
                if (qb < nqb) {
                    f32x4 a, c;
#pragma unroll
                    for (int j = 0; j < 4; j++) { a[j] = w.dbacc[qb][kt][j]; c[j] = w.dbacc[qb][kt][4 + j]; }
                    // (plain stores: the reduction that follows then finds the tiles in the memory-side cache)
                    *reinterpret_cast<f32x4*>(dst + 32 * qb + 8 * g) = a;
                    *reinterpret_cast<f32x4*>(dst + 32 * qb + 8 * g + 4) = c;
                }
            }
        }
    }
}

// Key rows >= n read as `key_pad` (-inf for the bias, so padded keys drop out of the softmax).
template <class T>
__global__ void __launch_bounds__(256) transpose_pad_kernel(const T* src, int64_t sa, int64_t sn, int n, int npk, int r,
                                                            const uint8_t* live, T* dst, float key_pad) {
    __shared__ T tile[32][33];
    const int a = blockIdx.z;
    if (live && !live[a]) return;
    const int q0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < 32; i += 8) {
        const int q = q0 + i, k = k0 + tx;
        tile[i][tx] = (q < n && k < n) ? src[a * sa + (int64_t)q * sn + k] : (T)(k >= n ? key_pad : 0.f);
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8) {
        const int k = k0 + i, q = q0 + tx;
        if (k < npk && q < r) dst[((int64_t)a * npk + k) * r + q] = tile[tx][i];
    }
}

// dbias[h][q][k] = sum_g part[h][g][k][q]; dscale[h] = gate * sum_g part_dscale[h][g].
// A partial tile is npk x r floats, key-major; a workgroup sums 256 consecutive floats of it (64 lanes x 16 bytes:
// every load of a wavefront is one contiguous KB) over the partial tiles of a head.  Each of its 4 wavefronts takes
// every 4th tile, and the 4 sums are added in a fixed order, so results are bit-reproducible.
template <int DT>
__global__ void __launch_bounds__(256) reduce_kernel(const BwdParams p, int npk, int r, bool has_bias) {
    typedef typename Elem<DT>::E E;
    __shared__ f32x4 part[3][64];
    const int h = blockIdx.z;
    if (has_bias) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int64_t gs = (int64_t)npk * r;
        const int64_t flat = 4 * ((int64_t)blockIdx.x * 64 + lane);
        const float* src = p.part_dbias + ((int64_t)h * p.db_parts) * gs + flat;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (flat < gs) {
#pragma unroll 8
            for (int gi = wave; gi < p.db_parts; gi += 4) acc += *reinterpret_cast<const f32x4*>(src + gi * gs);
        }
        if (wave) part[wave - 1][lane] = acc;
        __syncthreads();
        if (wave == 0 && flat < gs) {
            acc = ((acc + part[0][lane]) + part[1][lane]) + part[2][lane];
            const int k = (int)(flat / r), q = (int)(flat % r);
            if (k < p.n) {
                E* dst = reinterpret_cast<E*>(p.dbias) + ((int64_t)h * p.n + q) * p.n + k;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (q + i < p.n) dst[(int64_t)i * p.n] = (E)acc[i];
            }
        }
    }
    if (p.scale_kind == FWA2_SCALE_TENSOR && blockIdx.x == 0) {
        float v = 0.f;
        for (int gi = threadIdx.x; gi < p.ds_parts; gi += 256) v += p.part_dscale[(int64_t)h * p.ds_parts + gi];
        __shared__ float red[256];
        red[threadIdx.x] = v;
        __syncthreads();
        for (int sft = 128; sft > 0; sft >>= 1) {
            if (threadIdx.x < sft) red[threadIdx.x] += red[threadIdx.x + sft];
            __syncthreads();
        }
        if (threadIdx.x == 0) {
            const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
            reinterpret_cast<E*>(p.dscale)[h] = (E)(ls <= kLn100 ? red[0] : 0.f);
        }
    }
}

// ---- host side -----------------------------------------------------------------
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

#if FWA2_HALF != 2
int backward_supported(int n) { return n >= 1; }
#endif

void dq_geometry(int n, int* waves, int* chunks);
hipError_t launch_backward_dq(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st);
int backward_dq_resident_supported(int n);
int backward_fused_supported(int n);

hipError_t launch_backward_fused(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st,
                                 int max_groups, int* parts_out);
hipError_t launch_backward_dq_resident(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st,
                                       int max_groups, int* ds_parts_out);

// Largest set of score tables the one-pass kernel may ask for (one 256 KB table per head and per (window, head) of
// a masked call); calls beyond it stay on bwd_kernel + the dq kernel, which stream bias and mask from key-major copies.
constexpr size_t kTableBudget = (size_t)96 << 20;

hipError_t launch_backward_one(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st, int max_groups,
                               int* groups_out);

struct BwdPlan {
    int waves, groups, npk, r, nqb_t, kt, dq_waves, dq_chunks, ds_parts, dq_max_groups;
    bool one_pass;  // 161 .. 256 tokens: bwd_one_kernel (fwa2_bwd_one.hip) is the whole backward
    size_t off_tab;
    int n_chunks;   // > 1: windows of more than 256 tokens, cut into 256 x 256 or 192 x 192 super-tiles
    size_t off_dbias, off_dscale, off_bias_t, off_mask_t, off_delta, off_dk, off_dv, total;
    size_t smem;
};

static BwdPlan make_plan(int heads, int n, int bw, bool has_bias, bool has_mask, int n_windows, int cus) {
    BwdPlan pl;
    const int nqb = (n + 31) / 32;
    pl.n_chunks = (n + 255) / 256;
    pl.one_pass = false;
    int wg_per_cu;
    if (pl.n_chunks > 1) {
        // every workgroup is a full super-tile kernel of 256 x 256, or of 192 x 192 where that pads the
        // window less (576 = 3 x 192 tokens: 9 exact tiles instead of 9 tiles covering 768 x 768);
        // npk / r are the padded totals
        const int c192 = (n + 191) / 192;
        const int tile = 192 * c192 < 256 * pl.n_chunks ? 192 : 256;
        if (tile == 192) pl.n_chunks = c192;
        pl.nqb_t = tile / 32;
        pl.kt = 2;
        pl.waves = tile / 32;
        pl.npk = pl.r = tile * pl.n_chunks;
        wg_per_cu = 1;
    } else {
        pl.nqb_t = nqb <= 2 ? 2 : (nqb <= 4 ? 4 : (nqb == 5 ? 5 : 8));   // 5: 129 .. 160 tokens, tiles of 160 rows
        pl.r = 32 * pl.nqb_t;
        // up to 160 queries a wavefront owns one 16-key tile (<= 128 registers; several workgroups
        // per CU up to 128 queries, and at 129 .. 160 nine or ten wavefronts instead of five, which
        // measured 15 % faster at 144 tokens); above that two tiles (<= 256 registers, one workgroup
        // of up to 8 wavefronts per CU)
        pl.kt = nqb <= 5 ? 1 : 2;
        pl.waves = (n + 16 * pl.kt - 1) / (16 * pl.kt);
        pl.npk = pl.waves * 16 * pl.kt;
        wg_per_cu = pl.nqb_t == 2 ? 4 : (pl.nqb_t == 4 ? 2 : 1);
        const size_t slots = (size_t)heads * (1 + (has_mask ? n_windows : 0));
        if (pl.nqb_t == 8 && slots * 256 * 256 * 4 <= kTableBudget) {
            // four wavefronts of four key tiles on 256 x 256 tiles whatever the window length
            pl.one_pass = true;
            pl.kt = 4;
            pl.waves = 4;
            pl.npk = 256;
        }
    }
    int groups = (cus * wg_per_cu) / (heads * pl.n_chunks * pl.n_chunks);
    if (groups < 1) groups = 1;
    if (groups > bw) groups = bw;
    pl.groups = groups;
    size_t off = 0;
    pl.off_dbias = off;
    // one partial tile per workgroup and launch: two launches (masked / unmasked units) of bwd_kernel, one of the others
    if (has_bias) off += align256((size_t)heads * (pl.one_pass ? 1 : 2) * groups * pl.npk * pl.r * 4);
    dq_geometry(n, &pl.dq_waves, &pl.dq_chunks);
    pl.ds_parts = bw * pl.dq_chunks;
    // the resident dq kernel writes one partial per workgroup: at most this many per head and launch
    pl.dq_max_groups = (cus * 8) / heads + 1;
    if (pl.dq_max_groups > bw) pl.dq_max_groups = bw;
    const int ds_slots = pl.ds_parts > 2 * pl.dq_max_groups ? pl.ds_parts : 2 * pl.dq_max_groups;
    pl.off_dscale = off;
    off += align256((size_t)heads * ds_slots * 4);
    pl.off_delta = off;
    if (pl.n_chunks == 1 && !pl.one_pass) off += align256((size_t)bw * heads * pl.r * 4);
    pl.off_dk = off;
    if (pl.n_chunks > 1) off += align256((size_t)pl.n_chunks * bw * heads * pl.npk * 32 * 4);
    pl.off_dv = off;
    if (pl.n_chunks > 1) off += align256((size_t)pl.n_chunks * bw * heads * pl.npk * 32 * 4);
    pl.off_bias_t = off;
    if (has_bias && !pl.one_pass) off += align256((size_t)heads * pl.npk * pl.r * 2);
    pl.off_mask_t = off;
    if (has_mask && !pl.one_pass) off += align256((size_t)n_windows * pl.npk * pl.r * 4);
    pl.off_tab = off;
    if (pl.one_pass) off += align256((size_t)heads * (1 + (has_mask ? n_windows : 0)) * 256 * 256 * 4);
    pl.total = off;
    pl.smem = 0;   // the kernels use static LDS
    return pl;
}

#if FWA2_HALF != 2
size_t backward_workspace_bytes(int heads, int n, int bw, bool has_bias, bool has_mask, int n_windows, int cus) {
    if (!backward_supported(n)) return 0;
    return make_plan(heads, n, bw, has_bias, has_mask, n_windows, cus).total;
}
#endif

template <int DT, bool HAS_BIAS, int MASK_DT, int NQB, int KT, bool BIG, bool MAPPED = false>
static hipError_t launch_main(BwdParams p, const BwdPlan& pl, hipStream_t st, int* groups_out) {
    // Up to 64 tokens one launch walks masked and unmasked units alike; above that the two copies of
    // the block sequence cost occupancy (128 tokens) or spill (256), and each kind gets a launch.
    constexpr bool kOneLaunch = MASK_DT >= 0 && NQB <= 2 && !BIG;
    // asked once per device and block size (the wavefront count follows the window length)
    static std::atomic<int> fit_by_waves[17][3][kFitDevices];
    const int wslot = pl.waves <= 16 ? pl.waves : 0;
    int fit;
    if constexpr (kOneLaunch) {
        fit = resident_per_cu_cached(bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 2, BIG, MAPPED>, 64 * pl.waves, fit_by_waves[wslot][2]);
    } else {
        const int a = resident_per_cu_cached(bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 0, BIG, MAPPED>, 64 * pl.waves, fit_by_waves[wslot][0]);
        const int b = MASK_DT >= 0 ? resident_per_cu_cached(bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 1, BIG, MAPPED>, 64 * pl.waves,
                                                            fit_by_waves[wslot][1])
                                   : a;
        fit = a < b ? a : b;
    }
    const int tiles = pl.n_chunks * pl.n_chunks;
    // never more workgroups per head (and super-tile) than the plan sized the workspace for
    int groups = (p.cus * fit) / (p.heads * tiles);
    if (groups < 1) groups = 1;
    if (groups > pl.groups) groups = pl.groups;
    p.groups = groups;
    const bool two = !kOneLaunch && MASK_DT >= 0 && p.mask_live != nullptr;
    p.db_parts = two ? 2 * groups : groups;
    p.db_slot0 = 0;
    p.big_xcd = BIG && (p.heads * groups) % 8 == 0;       // super-tiles of a (head, group) pair on one XCD, see the kernel
    const dim3 grid(p.heads * tiles * groups), block(64 * pl.waves);
    if (p.ev_start) (void)hipEventRecord(p.ev_start, st);
    if constexpr (kOneLaunch) {
        hipLaunchKernelGGL((bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 2, BIG, MAPPED>), grid, block, 0, st, p);
    } else {
        // the units whose mask is all zero (or every unit when there is no mask) ...
        if (MASK_DT < 0 || two) hipLaunchKernelGGL((bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 0, BIG, MAPPED>), grid, block, 0, st, p);
        // ... and the units whose mask is live (all of them when the flags are absent)
        if (MASK_DT >= 0) {
            p.db_slot0 = two ? groups : 0;
            hipLaunchKernelGGL((bwd_kernel<DT, HAS_BIAS, MASK_DT, NQB, KT, 1, BIG, MAPPED>), grid, block, 0, st, p);
        }
    }
    if (p.ev_stop) (void)hipEventRecord(p.ev_stop, st);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (groups_out) { groups_out[0] = groups; groups_out[1] = p.db_parts; }
    return hipSuccess;
}


template <int DT, bool HAS_BIAS, int MASK_DT>
static hipError_t launch_nqb(const BwdParams& p, const BwdPlan& pl, hipStream_t st, int* groups_out) {
    if (p.map.nw > 0 && pl.n_chunks == 1) {
        // windows of up to 64 tokens with a map go to the fused kernel; those of more than 256 run on the
        // super-tiled form below, which reads the map at run time
        if (pl.nqb_t == 2) return hipErrorInvalidValue;
        if (pl.nqb_t == 4) return launch_main<DT, HAS_BIAS, MASK_DT, 4, 1, false, true>(p, pl, st, groups_out);
        if (pl.kt == 1) return launch_main<DT, HAS_BIAS, MASK_DT, 5, 1, false, true>(p, pl, st, groups_out);
        return launch_main<DT, HAS_BIAS, MASK_DT, 8, 2, false, true>(p, pl, st, groups_out);
    }
    if (pl.n_chunks > 1 && pl.nqb_t == 6) return launch_main<DT, HAS_BIAS, MASK_DT, 6, 2, true>(p, pl, st, groups_out);
    if (pl.n_chunks > 1) return launch_main<DT, HAS_BIAS, MASK_DT, 8, 2, true>(p, pl, st, groups_out);
    if (pl.nqb_t == 2) return launch_main<DT, HAS_BIAS, MASK_DT, 2, 1, false>(p, pl, st, groups_out);
    if (pl.nqb_t == 4) return launch_main<DT, HAS_BIAS, MASK_DT, 4, 1, false>(p, pl, st, groups_out);
    if (pl.kt == 1) return launch_main<DT, HAS_BIAS, MASK_DT, 5, 1, false>(p, pl, st, groups_out);
    return launch_main<DT, HAS_BIAS, MASK_DT, 8, 2, false>(p, pl, st, groups_out);
}

template <int DT>
static hipError_t launch_bwd_dt(BwdParams p, bool has_bias, int mask_dt, hipStream_t st) {
    typedef typename Elem<DT>::E E;
    const BwdPlan pl = make_plan(p.heads, p.n, p.bw, has_bias, mask_dt >= 0, p.n_windows, p.cus);
    unsigned char* ws = reinterpret_cast<unsigned char*>(p.workspace);
    p.waves = pl.waves;
    p.groups = pl.groups;
    p.dq_waves = pl.dq_waves;
    p.dq_chunks = pl.dq_chunks;
    p.ds_parts = pl.ds_parts;
    p.part_dbias = reinterpret_cast<float*>(ws + pl.off_dbias);
    p.part_dscale = reinterpret_cast<float*>(ws + pl.off_dscale);
    p.bias_t = ws + pl.off_bias_t;
    p.mask_t = ws + pl.off_mask_t;
    p.delta = reinterpret_cast<float*>(ws + pl.off_delta);
    p.delta_stride = pl.r;
    p.n_chunks = pl.n_chunks;
    p.r_tot = pl.r;
    p.npk_tot = pl.npk;
    p.part_dk = reinterpret_cast<float*>(ws + pl.off_dk);
    p.part_dv = reinterpret_cast<float*>(ws + pl.off_dv);
    if (backward_fused_supported(p.n)) {
        // one pass over q, k, v, o, dO; no key-major side tables, no delta buffer
        int parts = 0;
        const int mg = pl.groups < pl.dq_max_groups ? pl.groups : pl.dq_max_groups;
        hipError_t ef = launch_backward_fused(p, DT, has_bias, mask_dt, st, mg, &parts);
        if (ef != hipSuccess) return ef;
        p.db_parts = parts;
        p.ds_parts = parts;
        if (has_bias || p.scale_kind == FWA2_SCALE_TENSOR) {
            dim3 gr(has_bias ? (pl.npk * pl.r + 255) / 256 : 1, 1, p.heads);
            hipLaunchKernelGGL(reduce_kernel<DT>, gr, dim3(256), 0, st, p, pl.npk, pl.r, has_bias);
            ef = hipGetLastError();
        }
        return ef;
    }
    p.tab = reinterpret_cast<const float*>(ws + pl.off_tab);
    const dim3 tgrid(pl.r / 32, (pl.npk + 31) / 32, 1);
    if (has_bias && !pl.one_pass) {
        dim3 gr(tgrid.x, tgrid.y, p.heads);
        hipLaunchKernelGGL(transpose_pad_kernel<E>, gr, dim3(256), 0, st, reinterpret_cast<const E*>(p.bias), p.bias_sh,
                           p.bias_sn, p.n, pl.npk, pl.r, (const uint8_t*)nullptr,
                           reinterpret_cast<E*>(const_cast<void*>(p.bias_t)), -INFINITY);
    }
    if (mask_dt >= 0 && !pl.one_pass) {
        dim3 gr(tgrid.x, tgrid.y, p.n_windows);
        if (mask_dt == FWA2_F32)
            hipLaunchKernelGGL(transpose_pad_kernel<float>, gr, dim3(256), 0, st, reinterpret_cast<const float*>(p.mask),
                               p.mask_sw, p.mask_sn, p.n, pl.npk, pl.r, p.mask_live,
                               reinterpret_cast<float*>(const_cast<void*>(p.mask_t)), 0.f);
        else
            hipLaunchKernelGGL(transpose_pad_kernel<E>, gr, dim3(256), 0, st, reinterpret_cast<const E*>(p.mask),
                               p.mask_sw, p.mask_sn, p.n, pl.npk, pl.r, p.mask_live,
                               reinterpret_cast<E*>(const_cast<void*>(p.mask_t)), 0.f);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int gr_out[2] = {pl.groups, pl.groups};
    if (pl.one_pass) {
        e = launch_backward_one(p, DT, has_bias, mask_dt, st, pl.groups, gr_out);
        if (e != hipSuccess) return e;
        p.groups = gr_out[0];
        p.db_parts = gr_out[1];
        p.ds_parts = gr_out[0];
        if (has_bias || p.scale_kind == FWA2_SCALE_TENSOR) {
            dim3 gr(has_bias ? (pl.npk * pl.r + 255) / 256 : 1, 1, p.heads);
            hipLaunchKernelGGL(reduce_kernel<DT>, gr, dim3(256), 0, st, p, pl.npk, pl.r, has_bias);
            e = hipGetLastError();
        }
        return e;
    }
    if (has_bias) {
        if (mask_dt < 0) e = launch_nqb<DT, true, -1>(p, pl, st, gr_out);
        else if (mask_dt == FWA2_F32) e = launch_nqb<DT, true, FWA2_F32>(p, pl, st, gr_out);
        else e = launch_nqb<DT, true, DT>(p, pl, st, gr_out);
    } else {
        if (mask_dt < 0) e = launch_nqb<DT, false, -1>(p, pl, st, gr_out);
        else if (mask_dt == FWA2_F32) e = launch_nqb<DT, false, FWA2_F32>(p, pl, st, gr_out);
        else e = launch_nqb<DT, false, DT>(p, pl, st, gr_out);
    }
    if (e != hipSuccess) return e;
    p.groups = gr_out[0];
    p.db_parts = gr_out[1];
    // (windows of more than 256 tokens: the fp32 dk / dv partials are summed inside the dq launch that follows)
    if (backward_dq_resident_supported(p.n)) {
        int parts = 0;
        e = launch_backward_dq_resident(p, DT, has_bias, mask_dt, st, pl.dq_max_groups, &parts);
        p.ds_parts = parts;
    } else {
        e = launch_backward_dq(p, DT, has_bias, mask_dt, st);
    }
    if (e != hipSuccess) return e;
    if (has_bias || p.scale_kind == FWA2_SCALE_TENSOR) {
        dim3 gr(has_bias ? (pl.npk * pl.r + 255) / 256 : 1, 1, p.heads);
        hipLaunchKernelGGL(reduce_kernel<DT>, gr, dim3(256), 0, st, p, pl.npk, pl.r, has_bias);
        e = hipGetLastError();
    }
    return e;
}

#if FWA2_HALF == 2
hipError_t launch_backward_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    return launch_bwd_dt<FWA2_F16>(p, has_bias, mask_dt, st);
}
#else
#if FWA2_HALF == 1
hipError_t launch_backward_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st);
#endif
hipError_t launch_backward(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    if (dtype == FWA2_BF16) return launch_bwd_dt<FWA2_BF16>(p, has_bias, mask_dt, st);
#if FWA2_HALF == 1
    return launch_backward_f16(p, has_bias, mask_dt, st);
#else
    return launch_bwd_dt<FWA2_F16>(p, has_bias, mask_dt, st);
#endif
}
#endif

}  // namespace fwa2
