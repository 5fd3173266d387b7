// Backward, key side, for windows of up to 256 tokens: dk, dv, dbias and delta on gfx950.
//
// Replaces _bwd_preprocess_do_o_dot and the dK / dV / dbias half of _bwd_kernel of the reference
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:6-51, 84-353); dq comes from the query-side kernel.
//
// One workgroup of four wavefronts is persistent for one head, walks over many (batch*window) units and keeps
// the head's whole dbias tile in accumulator registers: every wavefront owns 64 keys (four MFMA tiles of 16)
// and streams the unit's queries past them in blocks of 32.  One wavefront per SIMD has 512 registers: the
// dbias accumulators (256 per lane) sit in AGPRs, the last quarter of them in LDS, and are only ever touched by
// the matrix pipe (dbias += I * dZ, an MFMA against a one-hot operand), which leaves the architectural
// registers to a software pipeline:
//
//   - bias and mask come as ONE fp32 table per head (per (window, head) where the window's mask is live) that
//     holds (bias + mask) * log2e in the order of the score accumulators, so the values of a block are loaded
//     straight into the C operand of S = Q_hat K_hat^T, one block ahead, into the registers the running
//     block has just read;
//   - the rows of Q_hat and dO and -delta of a block are read from LDS as soon as the block before it has issued
//     its last score product;
//   - the rows of the next unit's queries (q, dO, o, lse) travel global memory -> LDS (global_load_lds) in small
//     portions spread over the blocks of the current unit; the wavefront's own k and v rows are loaded into
//     registers behind the last block;
//   - per score the VALU does: add -lse, exp2, multiply by (dP - delta), two half conversions.
//
// Per unit:  landing rows -> tiles (q_hat * s * log2e in the score type, dO as is, -delta, -lse * log2e; each
// wavefront normalises its own 64 keys in registers), 8 blocks, then dk = (dk_hat - k_hat (dk_hat . k_hat)) / |k|
// and dv from registers.
#include <atomic>

#include "fwa2_common.hpp"

// FWA2_HALF splits this translation unit for the build: 0 the whole file; 1 everything except the fp16
// instantiations, which it reaches through launch_backward_key_f16(); 2 the fp16 instantiations alone.
#ifndef FWA2_HALF
#define FWA2_HALF 0
#endif

namespace fwa2 {

namespace key256 {

constexpr int kRow = 40;      // LDS row stride of the 16-bit tiles, in elements (80 bytes)
constexpr int R = 256;        // padded rows (queries and keys) of a unit
constexpr int NQB = 8;        // query blocks of 32
constexpr int KT = 4;         // key tiles of 16 per wavefront
constexpr int WAVES = 4;
constexpr int NT = 64 * WAVES;
// The 256 dbias accumulators of a lane are exactly the AGPR file, and the compiler needs a few AGPRs of its own
// (what it cannot hold in 256 VGPRs, it parks there with a register move; without room it spills to scratch,
// and a scratch reload queues behind every fetch in flight).  The accumulators of the last query block
// therefore live in LDS, in a private 16-byte slot per lane, and visit registers once per unit (two blocks:
// with one, some instantiations still spill).
constexpr int kLdsQb = 2;
__host__ __device__ constexpr bool db_in_lds(int qb) { return qb >= NQB - kLdsQb; }
constexpr int kLive = 256;    // windows whose mask flags are listed in LDS (more: every window counts as live)

template <class E>
__device__ __forceinline__ void async_row_chunk(const E* gsrc, E* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, kStreamPolicy);
}

// sum of squares / dot product of 8 elements, two at a time on the dot unit
__device__ __forceinline__ float dot8(bf16x8 a, bf16x8 b) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v2 x, y;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1]; y[0] = b[2 * j]; y[1] = b[2 * j + 1];
        s = __builtin_amdgcn_fdot2_f32_bf16(x, y, s, false);
    }
    return s;
}
__device__ __forceinline__ float dot8(f16x8 a, f16x8 b) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v2 x, y;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1]; y[0] = b[2 * j]; y[1] = b[2 * j + 1];
        s = __builtin_amdgcn_fdot2(x, y, s, false);
    }
    return s;
}

// Vector-memory instructions the compiler's wait-count bookkeeping must not see.  With a load into LDS or a store
// pending next to ordinary loads, the compiler no longer counts (returns of different kinds are not ordered for
// it) and puts s_waitcnt vmcnt(0) in front of the next use of a loaded table value, which then waits for rows
// that were requested from HBM a moment ago.  Issued from inline assembly they are invisible to it; its counted
// waits for the table loads then cover the hidden instructions too where those are older (returns are in order)
// and are merely stricter than needed where they are younger.  Whoever reads what these instructions wrote waits
// with an explicit s_waitcnt.  The compiler does not know these are memory instructions either, so the wait
// states it would put around them are part of the assembly: five between a VALU write of an SGPR (a
// v_readfirstlane behind the base or the LDS address) and the memory instruction that reads it, one after the
// write of M0, two after a 16-byte store before its data registers may be overwritten.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// 16 bytes per lane global -> LDS: lane i reads base + voff and lands at lds + 16 i (lds: wavefront-uniform)
__device__ __forceinline__ void vm_dma16(const void* base, uint32_t voff, uint32_t lds) {
    asm volatile("s_nop 3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}
// 4 bytes per lane: lands at lds + 4 i
__device__ __forceinline__ void vm_dma4(const void* base, uint32_t voff, uint32_t lds) {
    asm volatile("s_nop 3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1 nt" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}
#pragma clang diagnostic pop
// 16 bytes per lane, only from the lanes with idx < limit (exec is narrowed inside, so no branch splits the caller)
template <class V8, class E>
__device__ __forceinline__ void vm_store16_if_below(E* dst, V8 v, int idx, int limit) {
    uint64_t saved;
    asm volatile("v_cmp_lt_i32 vcc, %3, %4\n\ts_and_saveexec_b64 %0, vcc\n\tglobal_store_dwordx4 %1, %2, off nt\n\ts_nop 1\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(dst), "v"(v), "v"(idx), "s"(limit)
                 : "memory", "vcc", "scc");
}
__device__ __forceinline__ void vm_store4(float* dst, float v) {
    asm volatile("global_store_dword %0, %1, off" ::"v"(dst), "v"(v) : "memory");
}

// 1 / max(|x|, eps) from the sum of squares
__device__ __forceinline__ float inv_norm_fast(float sumsq) {
    return __builtin_amdgcn_rsqf(fmaxf(sumsq, kNormEps * kNormEps));
}

}  // namespace key256

// HAS_BIAS: dbias is wanted.  HAS_TAB: a table of (bias + mask) * log2e exists (always when there is a bias, a mask
// or padded keys).  MASKED: some units take the table of their (window, head) instead of the head's.
template <int DT, bool HAS_BIAS, bool HAS_TAB, bool MASKED, bool MAPPED>
__global__ void __launch_bounds__(key256::NT) bwd_key_kernel(const BwdParams p) {
    using namespace key256;
    constexpr int SDT = kScoreDT;
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<SDT>::E SE;
    typedef typename Elem<SDT>::V8 SV8;
    typedef typename Elem<DT>::V4 V4;

    const int h = blockIdx.x / p.groups;
    const int grp = blockIdx.x - h * p.groups;
    const int N = p.n;

    __shared__ __attribute__((aligned(16))) SE lds_Qs[R * kRow];
    __shared__ __attribute__((aligned(16))) E lds_dOs[R * kRow];
    __shared__ __attribute__((aligned(16))) float lds_nlse2[R];
    __shared__ __attribute__((aligned(16))) float lds_ndelta[R];
    __shared__ __attribute__((aligned(16))) E lds_rawQ[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawDO[R * 32];
    __shared__ __attribute__((aligned(16))) E lds_rawO[R * 32];
    __shared__ __attribute__((aligned(16))) float lds_rawLse[R];
    __shared__ float lds_dummy[NT];
    __shared__ __attribute__((aligned(16))) float lds_db[HAS_BIAS ? kLdsQb * KT * 2 * NT * 4 : 4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, g = lane >> 4;

    float s_true;
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float ls = (float)reinterpret_cast<const E*>(p.logit_scale)[h];
        s_true = expf(fminf(ls, kLn100));
    } else {
        s_true = p.default_scale;
    }
    const float scale2 = s_true * kLog2e;

    // dbias accumulators: register (half, i) of tile (qb, kt) belongs to query 32 qb + 16 half + 4 g + i, key 64 wave + 16 kt + l16
    f32x4 dbq[NQB][KT][2];
    SV8 sel[2];     // sel[half][m][k] = [k == 16 half + m]: lane (g, m) holds k = 8 g .. 8 g + 7
    if (HAS_BIAS) {
#pragma unroll
        for (int a = 0; a < NQB; a++)
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int hf = 0; hf < 2; hf++)
#pragma unroll
                    for (int i = 0; i < 4; i++) dbq[a][kt][hf][i] = 0.f;
#pragma unroll
        for (int i = 0; i < kLdsQb * KT * 2; i++) *reinterpret_cast<f32x4*>(lds_db + (i * NT + tid) * 4) = dbq[0][0][0];
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int j = 0; j < 8; j++) sel[hf][j] = (g == 2 * hf + (l16 >> 3) && j == (l16 & 7)) ? (SE)1.0f : (SE)0.0f;
    }

    // ---- the order in which the head's units are dealt out: the windows with a live mask first, window by
    // window (workgroups running side by side then share a table in the L2), then the others image by image ----
    __shared__ uint8_t lds_live[kLive];
    __shared__ uint16_t lds_list[kLive];
    __shared__ int lds_count;
    const bool listed = MASKED && p.mask_live && p.n_windows <= kLive;
    if (listed) {
        for (int i = tid; i < p.n_windows; i += NT) lds_live[i] = p.mask_live[i];
        __syncthreads();
        if (wave == 0) {
            int cnt = 0;
#pragma unroll 1
            for (int cls = 1; cls >= 0; cls--) {
                for (int base = 0; base < p.n_windows; base += 64) {
                    const int w = base + lane;
                    const bool in = w < p.n_windows && ((lds_live[w] != 0) == (cls != 0));
                    const unsigned long long bal = __ballot(in);
                    if (in) lds_list[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = (uint16_t)w;
                    cnt += __popcll(bal);
                }
                if (cls == 1 && lane == 0) lds_count = cnt;
            }
        }
        __syncthreads();
    }
    const int n_live = listed ? __builtin_amdgcn_readfirstlane(lds_count) : 0;
    const int n_img = (p.bw + p.n_windows - 1) / p.n_windows;
    const int t_live = listed ? n_img * n_live : (MASKED ? p.bw : 0);
    const int t_end = listed ? n_img * p.n_windows : p.bw;
    auto unit_of = [&](int t) -> int {
        if (!listed) return t;
        int img, wi;
        if (t < t_live) {
            wi = t / n_img;
            img = t - wi * n_img;
        } else {
            const int n_rest = p.n_windows - n_live;
            const int u = t - t_live;
            img = u / n_rest;
            wi = n_live + (u - img * n_rest);
        }
        return __builtin_amdgcn_readfirstlane(img * p.n_windows + (int)lds_list[wi]);
    };
    auto rank_from = [&](int t) -> int {
        for (; t < t_end; t += p.groups)
            if (unit_of(t) < p.bw) return t;
        return t_end;
    };
    // table of a unit: [key tile][query block][t][lane][4]; this wavefront's four key tiles, this lane's slot
    auto table_of = [&](int t, int b) -> const float* {
        const bool live = MASKED && t < t_live;
        const int slot = live ? p.heads + (b % p.n_windows) * p.heads + h : h;
        return p.tab + (int64_t)slot * (R * R) + ((wave * KT * NQB * 2) << 8);     // wavefront-uniform; the lane adds 4 * lane
    };
    const int lane4 = 4 * lane;

    // ---- rows of one unit, global memory -> landing area.  Every wavefront moves rows 64 wave .. 64 wave + 63 of
    // q, dO, o (16 rows per instruction) and of lse: 13 instructions, issued in portions of 2.  Rows beyond n
    // re-read row n - 1 (the tile builder zeroes them), so every instruction is issued with all lanes, without a
    // branch.  The instructions are hidden from the compiler's wait-count bookkeeping (see vm_* above). ----
    auto fetch_rows = [&](int b, int part) __attribute__((always_inline)) {
        // the lane index is re-derived on the spot (two instructions) wherever row addresses are formed, so that
        // the compiler does not keep dozens of lane-dependent address parts alive (or in scratch) across the unit loop
        const int lane = lane_now();
        const int dc = (lane & 3) * 8;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int idx = 2 * part + i;        // 0 .. 13
            if (idx < 12) {
                const int arr = idx >> 2;        // q, dO, o
                const int row0 = 64 * wave + 16 * (idx & 3);
                const int r = min(row0 + (lane >> 2), N - 1);
                const T4& t4 = arr == 0 ? p.q : arr == 1 ? p.d_o : p.o;
                E* dst = arr == 0 ? lds_rawQ : arr == 1 ? lds_rawDO : lds_rawO;
                const E* unit = unit_ptr<MAPPED, E>(t4, p.map, b, h);
                const uint32_t voff = (uint32_t)(reinterpret_cast<const char*>(row_at(unit, unit_row<MAPPED>(p.map, b, r), t4.sn, dc)) -
                                                 reinterpret_cast<const char*>(unit));
                vm_dma16(unit, voff, lds_addr(dst + row0 * 32));
            } else if (idx == 12) {
                const int r = min(64 * wave + lane, N - 1);
                vm_dma4(p.lse + b * p.lse_sb + h * p.lse_sh, 4u * (uint32_t)r, lds_addr(lds_rawLse + 64 * wave));
            }
        }
    };

    // The rows of the wavefront's own keys (k and v, 16 bytes per lane and key tile) skip the landing area: they
    // are requested after the last block of a unit and used after the next unit's tiles have been built.
    V8 kraw[KT], vraw[KT];
    auto fetch_keys = [&](int b) __attribute__((always_inline)) {
        const int ln = lane_now();
        const int l16 = ln & 15, g = ln >> 4;
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int key = min(64 * wave + 16 * kt + l16, N - 1);
            kraw[kt] = ld8<V8>(row_ptr<MAPPED, E>(p.k, p.map, b, h, key, 8 * g));
            vraw[kt] = ld8<V8>(row_ptr<MAPPED, E>(p.v, p.map, b, h, key, 8 * g));
        }
    };

    // The walk over the units is computed one unit ahead of its use, in the middle of the block loop, where its
    // scalar work (a few integer divisions) hides between the vector instructions.
    struct Unit { int t, b; const float* tab; };
    auto unit_at = [&](int t) -> Unit {
        Unit u;
        u.t = rank_from(t);
        u.b = u.t < t_end ? unit_of(u.t) : 0;
        u.tab = (HAS_TAB && u.t < t_end) ? table_of(u.t, u.b) : nullptr;
        return u;
    };
    Unit cur = unit_at(grp);
    Unit nxt = cur.t < t_end ? unit_at(cur.t + p.groups) : cur;
    f32x4 tb[KT][2];       // table values of the coming block: every register is refilled as soon as its product has read it
    if (cur.t < t_end) {
        if (HAS_TAB) {
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int tt = 0; tt < 2; tt++) tb[kt][tt] = *reinterpret_cast<const f32x4*>(cur.tab + lane4 + (((kt * NQB) * 2 + tt) << 8));
        }
#pragma unroll
        for (int part = 0; part < 7; part++) fetch_rows(cur.b, part);
        fetch_keys(cur.b);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();

    while (cur.t < t_end) {
        const int b = cur.b;
        const bool have_next = nxt.t < t_end;
        // without a next unit the read-ahead fetches this one again: harmless, and the loop body stays free of branches
        const int b_next = have_next ? nxt.b : b;
        const float* tab = cur.tab;
        const float* tab_next = have_next ? nxt.tab : tab;
        Unit after = nxt;

        // ---- landing area -> tiles: q_hat * s * log2e, dO, -delta, -lse * log2e.  Thread = 8 columns of 4 rows.
        // Straight-line code: of every group of four lanes (one row), lane 0 writes -delta, lane 1 -lse * log2e and
        // the other two a dummy word, through one store whose address and value are selected per lane. ----
        {
            const int dc = (tid & 3) * 8;
            V8 q8[4], do8[4], o8[4];
            float lse_r[4];
#pragma unroll
            for (int it = 0; it < R / (NT / 4); it++) {
                const int r = (tid >> 2) + it * (NT / 4);
                q8[it] = ld8<V8>(lds_rawQ + r * 32 + dc);
                do8[it] = ld8<V8>(lds_rawDO + r * 32 + dc);
                o8[it] = ld8<V8>(lds_rawO + r * 32 + dc);
                lse_r[it] = lds_rawLse[r];
            }
#pragma unroll
            for (int it = 0; it < R / (NT / 4); it++) {
                const int r = (tid >> 2) + it * (NT / 4);
                if (N < R && r >= N) { q8[it] = zero8<V8>(); do8[it] = zero8<V8>(); }
                const float sq = quad_add(dot8(q8[it], q8[it]));
                const float dl = quad_add(dot8(o8[it], do8[it]));
                const float iq = inv_norm_fast(sq) * scale2;
                SV8 qn;
#pragma unroll
                for (int j = 0; j < 8; j++) qn[j] = (SE)((float)q8[it][j] * iq);
                st8<SV8>(lds_Qs + r * kRow + dc, qn);
                st8<V8>(lds_dOs + r * kRow + dc, do8[it]);
                const float l2 = (r < N && lse_r[it] != -INFINITY) ? -lse_r[it] * kLog2e : -INFINITY;   // padded / fully masked rows: P = 0
                const int role = tid & 3;
                float* dst = role == 0 ? lds_ndelta + r : role == 1 ? lds_nlse2 + r : lds_dummy + tid;
                *dst = role == 0 ? -dl : l2;
            }
        }
        // ---- this wavefront's keys: k_hat (score type) and v as B operands, 1 / |k| for the epilogue ----
        SV8 bk[KT];
        V8 bv[KT];
        float kinv[KT];     // negative: |k| <= eps, the projection term of the Jacobian is dropped
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int key = 64 * wave + 16 * kt + l16;
            V8 k8 = kraw[kt];
            bv[kt] = vraw[kt];
            if (N < R && key >= N) { k8 = zero8<V8>(); bv[kt] = zero8<V8>(); }
            const float sk = col_add(dot8(k8, k8));
            const float ik = inv_norm_fast(sk);
#pragma unroll
            for (int j = 0; j < 8; j++) bk[kt][j] = (SE)((float)k8[j] * ik);
            kinv[kt] = sk > kNormEps * kNormEps ? ik : -ik;
        }
        __syncthreads();   // tiles complete; the landing area is free again

        f32x4 dvacc[KT][2], dkacc[KT][2];
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
#pragma unroll
                for (int i = 0; i < 4; i++) { dvacc[kt][dt][i] = 0.f; dkacc[kt][dt][i] = 0.f; }

        // LDS operands of a block.  The rows of Q_hat and dO and -delta are only read by the S and dP products, so
        // their registers are refilled with the coming block's values as soon as the last such product of a block
        // has been issued; -lse and the transposed operands are read at the top of their block and arrive behind
        // the first products.
        SV8 aq[2];
        V8 ado[2];
        f32x4 nd[2];
        // lane parts of the LDS addresses; the block's part is a compile-time constant that folds into the instruction
        const int row_base = (8 * (l16 >> 2) + (l16 & 3)) * kRow + 8 * g;       // + (32 qb + 4 t) * kRow
        const int tr_base = (8 * g + (l16 >> 2)) * kRow + 8 * (l16 & 3);         // + 32 qb * kRow + 4 dt (+ 4 kRow)
        auto load_rows = [&](int qb) __attribute__((always_inline)) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                aq[tt] = ld8<SV8>(lds_Qs + row_base + (32 * qb + 4 * tt) * kRow);
                ado[tt] = ld8<V8>(lds_dOs + row_base + (32 * qb + 4 * tt) * kRow);
                nd[tt] = *reinterpret_cast<const f32x4*>(lds_ndelta + 8 * g + (32 * qb + 4 * tt));
            }
        };
        load_rows(0);

#pragma unroll
        for (int qb = 0; qb < NQB; qb++) {
            f32x4 nl[2];
            V8 tdo[2];
            SV8 tq[2];
#pragma unroll
            for (int tt = 0; tt < 2; tt++) nl[tt] = *reinterpret_cast<const f32x4*>(lds_nlse2 + 8 * g + (32 * qb + 4 * tt));
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4: the lane's dk / dv values are d = 8 g + 4 dt + i
                const int off = 32 * qb * kRow + 4 * dt;
                tdo[dt] = lds_tr8<DT>(lds_dOs + tr_base + off, lds_dOs + tr_base + off + 4 * kRow);
                tq[dt] = lds_tr8<SDT>(lds_Qs + tr_base + off, lds_Qs + tr_base + off + 4 * kRow);
            }
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
                f32x4 sacc[2], pacc[2];
#pragma unroll
                for (int tt = 0; tt < 2; tt++) {
                    // (S + bias + mask) * log2e with the table as the C operand; dP - delta
                    sacc[tt] = Elem<SDT>::mfma16(aq[tt], bk[kt], HAS_TAB ? tb[kt][tt] : nl[tt]);
                    pacc[tt] = Elem<DT>::mfma16(ado[tt], bv[kt], nd[tt]);
                }
                // the table registers are free again: refill them with the coming block's values (the last block
                // reads the first block of the next unit's table)
                if (HAS_TAB) {
                    const float* src = qb + 1 < NQB ? tab + (((kt * NQB + qb + 1) * 2) << 8) : tab_next + (((kt * NQB) * 2) << 8);
#pragma unroll
                    for (int tt = 0; tt < 2; tt++) tb[kt][tt] = *reinterpret_cast<const f32x4*>(src + lane4 + (tt << 8));
                }
                if (kt == KT - 1 && qb + 1 < NQB) load_rows(qb + 1);
                // everything read ahead is on its way before this tile's elementwise work starts
                asm volatile("" : "+v"(sacc[0]), "+v"(sacc[1]) :: "memory");
                // right behind the block's last batch of table loads (which then never queue behind rows requested
                // from HBM a moment ago): a portion of the next unit's rows; and once per unit delta for the dq kernel
                if (kt == KT - 1 && qb < 7) fetch_rows(b_next, qb);
                if (kt == 2 && qb == 3 && have_next) after = unit_at(nxt.t + p.groups);      // scalar work, off the critical path
                if (kt == 1 && qb == 0) {
                    const int r = 64 * wave + lane;
                    const float dl = -lds_ndelta[r];
                    vm_store4(p.delta + ((int64_t)b * p.heads + h) * p.delta_stride + r, dl);      // delta_stride = 256: rows beyond n are padding
                }
                V8 p8;
                SV8 z8;
#pragma unroll
                for (int tt = 0; tt < 2; tt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float x = HAS_TAB ? sacc[tt][i] + nl[tt][i] : sacc[tt][i];
                        const float pj = fast_exp2(x);
                        const float dz = pj * pacc[tt][i];
                        p8[4 * tt + i] = (E)pj;
                        z8[4 * tt + i] = (SE)dz;
                    }
                if (HAS_BIAS) {
#pragma unroll
                    for (int hf = 0; hf < 2; hf++) {
                        if (db_in_lds(qb)) {
                            f32x4* slot = reinterpret_cast<f32x4*>(lds_db + ((((qb - (NQB - kLdsQb)) * KT + kt) * 2 + hf) * NT + tid) * 4);
                            *slot = Elem<SDT>::mfma16(sel[hf], z8, *slot);
                        } else {
                            dbq[qb][kt][hf] = Elem<SDT>::mfma16(sel[hf], z8, dbq[qb][kt][hf]);
                        }
                    }
                }
#pragma unroll
                for (int dt = 0; dt < 2; dt++) {
                    dvacc[kt][dt] = Elem<DT>::mfma16(tdo[dt], p8, dvacc[kt][dt]);
                    dkacc[kt][dt] = Elem<SDT>::mfma16(tq[dt], z8, dkacc[kt][dt]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        fetch_keys(b_next);
        // ---- epilogue dk, dv: lane (key, g) holds d = 8 g + 4 dt + i, which is 16 bytes of a row ----
        const int ln_e = lane_now();
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int l16 = ln_e & 15, g = ln_e >> 4;
            const int key = 64 * wave + 16 * kt + l16;
            float x[8], a[8];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                x[j] = (float)bk[kt][j];
                a[j] = dkacc[kt][j >> 2][j & 3] * kLn2;      // undo the log2e folded into Q_hat
                dot += a[j] * x[j];
            }
            dot = col_add(dot);
            const float inv = fabsf(kinv[kt]);
            const float proj = kinv[kt] > 0.f ? dot : 0.f;
            V8 o8, v8;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                o8[j] = (E)(inv * (a[j] - x[j] * proj));
                v8[j] = (E)dvacc[kt][j >> 2][j & 3];
            }
            // keys beyond n (only with n < 256) address row n - 1 and are masked out of the store
            const int krow = min(key, N - 1);
            vm_store16_if_below(const_cast<E*>(row_ptr<MAPPED, E>(p.dk, p.map, b, h, krow)) + 8 * g, o8, key, N);
            vm_store16_if_below(const_cast<E*>(row_ptr<MAPPED, E>(p.dv, p.map, b, h, krow)) + 8 * g, v8, key, N);
        }
        cur = nxt;
        nxt = after;
        // The next unit's rows have landed once at most the youngest 16 vector-memory instructions are in flight:
        // the last portion of rows was issued in block 6; the 8 table loads of block 7, the 8 loads of the next
        // unit's keys (and the stores of the epilogue, which need not be waited for) are younger.
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        __syncthreads();   // ... everybody's rows; and every wavefront is done with the tiles
    }

    // ---- flush the per-workgroup partial sums: [head][partial][key][query] ----
    if (HAS_BIAS) {
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            float* dst = p.part_dbias + (((int64_t)h * p.db_parts + p.db_slot0 + grp) * R + 64 * wave + 16 * kt + l16) * R;
#pragma unroll
            for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    const f32x4 acc = db_in_lds(qb) ? *reinterpret_cast<const f32x4*>(
                                                          lds_db + ((((qb - (NQB - kLdsQb)) * KT + kt) * 2 + hf) * NT + tid) * 4)
                                                    : dbq[qb][kt][hf];
                    __builtin_nontemporal_store(acc, reinterpret_cast<f32x4*>(dst + 32 * qb + 16 * hf + 4 * g));
                }
        }
    }
}

// tab[slot][key tile j][query block qb][t][lane][i] = (bias[h][q][key] + mask[w][q][key]) * log2e with key = 16 j +
// lane % 16 and q = 32 qb + 8 (lane / 16) + 4 t + i: the order in which the 16 x 16 score accumulators of a wavefront
// hold a block; -inf for padded keys, 0 for padded queries.  Slot h < heads: the bias of head h alone; slot heads +
// w * heads + h: with the mask of window w (built only for windows whose mask is live; every window without flags).
template <class E, class ME>
__global__ void __launch_bounds__(256) build_table_kernel(const E* bias, int64_t bias_sh, int64_t bias_sn, const ME* mask,
                                                          int64_t mask_sw, int64_t mask_sn, const uint8_t* live, int n,
                                                          int heads, float* tab) {
    using namespace key256;
    const int slot = blockIdx.y;
    int h = slot, wnd = -1;
    if (slot >= heads) {
        wnd = (slot - heads) / heads;
        h = (slot - heads) - wnd * heads;
        if (live && !live[wnd]) return;
    }
    const int idx = blockIdx.x * 256 + threadIdx.x;        // (j, qb, t, lane)
    const int lane = idx & 63, t = (idx >> 6) & 1, rest = idx >> 7;
    const int qb = rest % NQB, j = rest / NQB;
    const int key = 16 * j + (lane & 15), q0 = 32 * qb + 8 * (lane >> 4) + 4 * t;
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int q = q0 + i;
        float x = 0.f;
        if (key >= n) {
            x = -INFINITY;
        } else if (q < n) {
            if (bias) x = (float)bias[h * bias_sh + (int64_t)q * bias_sn + key];
            if (wnd >= 0) x += (float)mask[wnd * mask_sw + (int64_t)q * mask_sn + key];
            x *= kLog2e;
        }
        v[i] = x;
    }
    *reinterpret_cast<f32x4*>(tab + (int64_t)slot * (R * R) + (int64_t)idx * 4) = v;
}

// ---- host side -----------------------------------------------------------------
template <int DT, bool HAS_BIAS, bool HAS_TAB, bool MASKED, bool MAPPED>
static hipError_t launch_key(BwdParams p, hipStream_t st, int max_groups, int* groups_out) {
    static std::atomic<int> fit_by_device[kFitDevices];
    const int fit = resident_per_cu_cached(bwd_key_kernel<DT, HAS_BIAS, HAS_TAB, MASKED, MAPPED>, key256::NT, fit_by_device);
    int groups = (p.cus * fit) / p.heads;
    if (groups < 1) groups = 1;
    if (groups > max_groups) groups = max_groups;
    p.groups = groups;
    p.db_parts = groups;
    p.db_slot0 = 0;
    hipLaunchKernelGGL((bwd_key_kernel<DT, HAS_BIAS, HAS_TAB, MASKED, MAPPED>), dim3(p.heads * groups), dim3(key256::NT), 0, st, p);
    if (groups_out) { groups_out[0] = groups; groups_out[1] = groups; }
    return hipGetLastError();
}

// The score tables of a call: slot h for every head, slot heads + w * heads + h for every window whose mask is live.
template <int DT>
static hipError_t build_tables(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st) {
    typedef typename Elem<DT>::E E;
    const bool masked = mask_dt >= 0;
    const bool has_tab = has_bias || masked || p.n < key256::R;
    if (!has_tab) return hipSuccess;
    const int slots = p.heads * (1 + (masked ? p.n_windows : 0));
    const dim3 gr(key256::R * key256::R / 4 / 256, slots);
    float* tab = const_cast<float*>(p.tab);
    const E* bias = reinterpret_cast<const E*>(p.bias);
    // The kernels list the flags of up to kLive windows; with more they treat every window as live and read
    // every window's table, so every table has to be built then, whatever the flags say.
    const uint8_t* live = p.n_windows <= key256::kLive ? p.mask_live : nullptr;
    if (mask_dt == FWA2_F32)
        hipLaunchKernelGGL((build_table_kernel<E, float>), gr, dim3(256), 0, st, bias, p.bias_sh, p.bias_sn,
                           reinterpret_cast<const float*>(p.mask), p.mask_sw, p.mask_sn, live, p.n, p.heads, tab);
    else
        hipLaunchKernelGGL((build_table_kernel<E, E>), gr, dim3(256), 0, st, bias, p.bias_sh, p.bias_sn,
                           reinterpret_cast<const E*>(p.mask), p.mask_sw, p.mask_sn, live, p.n, p.heads, tab);
    return hipGetLastError();
}

template <int DT>
static hipError_t launch_key_dt(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out) {
    const bool masked = mask_dt >= 0;
    const bool has_tab = has_bias || masked || p.n < key256::R;
    const bool mapped = p.map.nw > 0;
    hipError_t e = build_tables<DT>(p, has_bias, mask_dt, st);
    if (e != hipSuccess) return e;
    if (p.ev_start) (void)hipEventRecord(p.ev_start, st);
#define FWA2_KEY_CASE(B, T, M)                                                                                       \
    (mapped ? launch_key<DT, B, T, M, true>(p, st, max_groups, groups_out) : launch_key<DT, B, T, M, false>(p, st, max_groups, groups_out))
    if (has_bias) e = masked ? FWA2_KEY_CASE(true, true, true) : FWA2_KEY_CASE(true, true, false);
    else if (masked) e = FWA2_KEY_CASE(false, true, true);
    else if (has_tab) e = FWA2_KEY_CASE(false, true, false);
    else e = FWA2_KEY_CASE(false, false, false);
#undef FWA2_KEY_CASE
    if (p.ev_stop) (void)hipEventRecord(p.ev_stop, st);
    return e;
}

#if FWA2_HALF == 2
hipError_t launch_backward_key_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out) {
    return launch_key_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, groups_out);
}
#else
#if FWA2_HALF == 1
hipError_t launch_backward_key_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out);
#endif
// The tables alone, for the one-pass kernel (fwa2_bwd_one.hip), which reads them in the same order.
hipError_t launch_key_tables(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st) {
    return dtype == FWA2_BF16 ? build_tables<FWA2_BF16>(p, has_bias, mask_dt, st) : build_tables<FWA2_F16>(p, has_bias, mask_dt, st);
}

// dk, dv, delta and the dbias partial tiles of a call with 161 .. 256 tokens per window; p.tab points at room for
// heads * (1 + windows) tables of 256 x 256 floats.  groups_out: workgroups per head, partial tiles per head.
hipError_t launch_backward_key(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st, int max_groups,
                               int* groups_out) {
    if (dtype == FWA2_BF16) return launch_key_dt<FWA2_BF16>(p, has_bias, mask_dt, st, max_groups, groups_out);
#if FWA2_HALF == 1
    return launch_backward_key_f16(p, has_bias, mask_dt, st, max_groups, groups_out);
#else
    return launch_key_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, groups_out);
#endif
}
#endif

}  // namespace fwa2
