// Backward in ONE pass for windows of 161 .. 256 tokens on gfx950: dq, dk, dv, dbias, delta and the logit-scale
// terms from a single recomputation of the scores, reading q, k, v, o, dO once.
//
// Replaces _bwd_preprocess_do_o_dot and _bwd_kernel of the reference
// (flash_win_attn_v2/kernels/attn_kernel_backward.py:6-51, 84-353), which also recomputes every score once
// (:246-336) but sums dq and dbias with fp32 atomics; here nothing is atomic and every sum has a fixed order.
//
// One workgroup of four wavefronts (one per SIMD, 512 registers each) is persistent for one head, walks over many
// (batch*window) units and keeps the head's whole dbias tile on chip: every wavefront owns 64 keys (four MFMA tiles
// of 16) and the unit's queries stream past them in blocks of 32.  The dbias accumulators of a lane (256 floats)
// sit in AGPRs, the last quarter of them in LDS, and are only ever touched by the matrix pipe (dbias += I * dZ, an
// MFMA against a one-hot operand).  Bias and mask come as ONE fp32 table per head (per (window, head) where the
// window's mask is live; fwa2_score_tables.hip) that holds (bias + mask) * log2e in the order of the score
// accumulators, so the values of a block are loaded straight into the C operand of S = Q_hat K_hat^T, one block
// ahead, into the registers the running block has just read; masked and unmasked units run the same code in one
// launch.  Per score the VALU does: add -lse, exp2, multiply by (dP - delta), two half conversions.
//
// The blocks are a software pipeline over ALL the units the workgroup walks, with one barrier per block and no
// per-unit staging phase:
//
//   iteration of block X:   rows of block X+3      global memory -> landing slot (global_load_lds, 2 slots)
//                           block X+2              landing slot -> tiles (q_hat s log2e, dO, -delta, -lse log2e, 1/|q|; 4 slots)
//                           block X                S, dP, exp2, dZ, dbias, dV, dK_hat against the wavefront's keys; the
//                                                  wavefront's dZ (32 queries x 64 keys, fp16) also goes to its own
//                                                  LDS slab and comes back transposed (ds_read_b64_tr_b16) as the
//                                                  B operand of dQ_hat^T += K_hat^T dZ^T over its 64 keys
//                           block X                that partial dQ_hat (32 x 32 fp32) -> LDS (2 slots)
//                           block X-1              the four wavefronts' partials are summed (fixed order), taken
//                                                  back through q / max(|q|, eps), and stored; q_hat . dq_hat is the
//                                                  row's term of dlogit_scale
//
// so the landing area and the tiles hold a few blocks instead of a whole unit, which is what makes room in LDS
// for the dZ slabs and the dq partials next to the 64 KB of dbias accumulators that do not fit the registers.
#include <atomic>

#include "fwa2_common.hpp"

// FWA2_HALF splits this translation unit for the build: 0 the whole file; 1 everything except the fp16
// instantiations, which it reaches through launch_backward_one_f16(); 2 the fp16 instantiations alone.
#ifndef FWA2_HALF
#define FWA2_HALF 0
#endif

namespace fwa2 {

hipError_t launch_score_tables(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st);

namespace one256 {

constexpr int kRow = 40;      // LDS row stride of the 16-bit tiles, in elements (80 bytes)
constexpr int R = 256;        // padded rows (queries and keys) of a unit
constexpr int NQB = 8;        // query blocks of 32
constexpr int KT = 4;         // key tiles of 16 per wavefront
constexpr int WAVES = 4;
constexpr int NT = 64 * WAVES;
// The 256 dbias accumulators of a lane are exactly the AGPR file, and the compiler needs a few AGPRs of its own (what
// it cannot hold in 256 VGPRs, it parks there with a register move; without room it spills to scratch, and a scratch
// reload queues behind every fetch in flight).  The accumulators of the last query blocks therefore live in LDS, in
// a private 16-byte slot per lane, and visit registers once per unit (two blocks: with one, some instantiations
// still spill).
constexpr int kLdsQb = 2;
__host__ __device__ constexpr bool db_in_lds(int qb) { return qb >= NQB - kLdsQb; }
constexpr int kLive = 256;    // windows whose mask flags are listed in LDS (more: every window counts as live)
constexpr int kLandE = 3 * 32 * 32 + 512;   // elements of a landing slot: three tensors' rows and 1 KB for lse
constexpr int kPartRow = 36;  // floats per query row of a dq partial tile (32 + 4: rows 144 bytes apart)

// sum of squares / dot product of 4 elements, two at a time on the dot unit
__device__ __forceinline__ float dot4(bf16x4 a, bf16x4 b) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        v2 x, y;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1]; y[0] = b[2 * j]; y[1] = b[2 * j + 1];
        s = __builtin_amdgcn_fdot2_f32_bf16(x, y, s, false);
    }
    return s;
}
__device__ __forceinline__ float dot4(f16x4 a, f16x4 b) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        v2 x, y;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1]; y[0] = b[2 * j]; y[1] = b[2 * j + 1];
        s = __builtin_amdgcn_fdot2(x, y, s, false);
    }
    return s;
}
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

// Sum over the 8 lanes of an aligned group of eight: the quad sum, then the other quad's through a mirror of the
// half row (lane i <- lane 7 - i).
__device__ __forceinline__ float oct_add(float x) {
    x = quad_add(x);
    const float y = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x141, 0xF, 0xF, true));
    return x + y;
}

// Vector-memory instructions the compiler's wait-count bookkeeping must not see (it would guard every LDS read it
// cannot tell from the copies' targets with a wait for all of them): the copies
// into LDS and the output stores are issued from inline assembly, and whoever reads what the copies wrote waits
// with an explicit s_waitcnt.  Loads return in order, so "at most n loads outstanding" means everything older
// than the youngest n loads has arrived; outstanding stores only make such a wait stricter.
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
// 16 / 8 bytes per lane, only from the lanes with idx < limit (exec is narrowed inside, so no branch splits the caller)
template <class V8, class E>
__device__ __forceinline__ void vm_store16_if_below(E* dst, V8 v, int idx, int limit) {
    uint64_t saved;
    asm volatile("v_cmp_lt_i32 vcc, %3, %4\n\ts_and_saveexec_b64 %0, vcc\n\tglobal_store_dwordx4 %1, %2, off nt\n\ts_nop 1\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(dst), "v"(v), "v"(idx), "s"(limit)
                 : "memory", "vcc", "scc");
}
template <class V4, class E>
__device__ __forceinline__ void vm_store8_if_below(E* dst, V4 v, int idx, int limit) {
    uint64_t saved;
    asm volatile("v_cmp_lt_i32 vcc, %3, %4\n\ts_and_saveexec_b64 %0, vcc\n\tglobal_store_dwordx2 %1, %2, off nt\n\ts_nop 1\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(dst), "v"(v), "v"(idx), "s"(limit)
                 : "memory", "vcc", "scc");
}

// 16 bytes per lane at base + voff (base: wavefront-uniform); two wait states before the data registers may change
template <class V8>
__device__ __forceinline__ void vm_store16(void* base, uint32_t voff, V8 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1" ::"v"(voff), "v"(v), "s"(base) : "memory");
}
// 8 bytes per lane at base + voff (base: wavefront-uniform)
template <class V4>
__device__ __forceinline__ void vm_store8(void* base, uint32_t voff, V4 v) {
    asm volatile("global_store_dwordx2 %0, %1, %2 nt" ::"v"(voff), "v"(v), "s"(base) : "memory");
}

// 1 / max(|x|, eps) from the sum of squares
__device__ __forceinline__ float inv_norm_fast(float sumsq) {
    return __builtin_amdgcn_rsqf(fmaxf(sumsq, kNormEps * kNormEps));
}

}  // namespace one256

// HAS_BIAS: dbias is wanted.  HAS_TAB: a table of (bias + mask) * log2e exists (always when there is a bias, a mask
// or padded keys).  MASKED: some units take the table of their (window, head) instead of the head's.  ROWS: how
// rows are addressed -- 0 any window length without a window map, 1 through the window map, 2 windows of exactly
// 256 tokens without a map (every block is whole: no clamping, no predicated stores, no branches in the copies).
template <int DT, bool HAS_BIAS, bool HAS_TAB, bool MASKED, int ROWS>
__global__ void __launch_bounds__(one256::NT) bwd_one_kernel(const BwdParams p) {
    using namespace one256;
    constexpr bool MAPPED = ROWS == 1;
    constexpr bool PLAIN = ROWS == 2;
    constexpr int SDT = kScoreDT;
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    typedef typename Elem<DT>::V4 V4;
    typedef typename Elem<SDT>::E SE;
    typedef typename Elem<SDT>::V8 SV8;
    typedef typename Elem<SDT>::V4 SV4;

    const int h = blockIdx.x / p.groups;
    const int grp = blockIdx.x - h * p.groups;
    const int N = PLAIN ? R : p.n;      // whole 256-token windows: a compile-time constant

    // landing slots (block X & 1): 32 rows of q, dO, o as they are in memory, and their lse
    // (per slot: q, dO, o rows, 2 KB each, then 1 KB for the lse values: what wavefront w copies lands 2 KB x w
    // into the slot)
    __shared__ __attribute__((aligned(16))) E lds_raw[2][kLandE];
    // tile slots (block X & 3)
    __shared__ __attribute__((aligned(16))) SE lds_Qs[4][32 * kRow];
    __shared__ __attribute__((aligned(16))) E lds_dOs[4][32 * kRow];
    // per tile slot: -delta, -lse * log2e, 1 / |q| of its 32 rows, and a row nobody reads
    __shared__ __attribute__((aligned(16))) float lds_meta[4][4][32];
    // per wavefront: dZ of the running block, [key of the wavefront][query of the block] (also K_hat once per unit)
    __shared__ __attribute__((aligned(16))) SE lds_zst[WAVES][64 * kRow];
    // dQ_hat partials (block X & 1) of the four wavefronts, [query][d] fp32
    __shared__ __attribute__((aligned(16))) float lds_part[2][WAVES][32 * kPartRow];
    __shared__ float lds_red[WAVES];
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
    const float unscale = 1.0f / scale2;

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

    // Wavefront-uniform start of unit b inside a tensor whose head offset is already part of `base`.
    auto unit_start = [&](const char* base, int64_t sb, int b) -> const char* {
        return base + (int64_t)(MAPPED ? b / p.map.nw : b) * sb * (int64_t)sizeof(E);
    };
    // ---- rows of block qb of unit b, global memory -> landing slot.  Wavefront 0 moves the 32 rows of q (16 per
    // instruction), 1 those of dO, 2 those of o, 3 the lse values (twice, so that every wavefront has issued the
    // same number of copies).  Rows beyond n re-read row n - 1 (the tile builder zeroes them).  What a wavefront
    // copies never changes, so its tensor is picked once. ----
    const T4& mine = wave == 0 ? p.q : wave == 1 ? p.d_o : p.o;
    const char* const mine_base = reinterpret_cast<const char*>(mine.ptr) + (int64_t)h * mine.sh * (int64_t)sizeof(E);
    const int64_t mine_sb = mine.sb, mine_sn = mine.sn;
    const float* const lse_base = p.lse + h * p.lse_sh;
    const int meta_lane = min(tid & 7, 3) * 32 + (tid >> 3);
    // Whole blocks without a window map (PLAIN): a lane's byte offset into its source is a constant of the lane
    // plus a scalar of the block, and wavefront 3 copies its 128 bytes of lse with the same 16-byte instruction
    // (8 lanes' worth, repeated), so the copies are the same two instructions in every wavefront.
    const uint32_t mine_lane = wave < 3 ? (uint32_t)(((lane >> 2) * (int)mine_sn + (lane & 3) * 8) * (int)sizeof(E)) : 16u * (uint32_t)(lane & 7);
    const uint32_t mine_blk = wave < 3 ? (uint32_t)(32 * (int)mine_sn * (int)sizeof(E)) : 128u;      // one block further on
    const uint32_t mine_half = wave < 3 ? mine_blk / 2 : 0u;                                          // its second 16 rows
    const uint32_t land_wave = lds_addr(&lds_raw[0][0]) + 2048u * (uint32_t)wave;
    const uint32_t land_half = wave < 3 ? 1024u : 0u;
    // the wavefront's source inside unit b: its tensor's rows, or the unit's lse values
    auto source_of = [&](int b) -> const char* {
        return wave < 3 ? unit_start(mine_base, mine_sb, b) : reinterpret_cast<const char*>(lse_base + b * p.lse_sb);
    };
    auto dma_block = [&](const char* src, int b, int qb, int slot) __attribute__((always_inline)) {
        if (PLAIN) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                uint32_t voff = mine_lane, blk = mine_blk, half = mine_half, dst = land_wave, dhalf = land_half;
                // taken as opaque here: one add per copy instead of a register per block and slot kept across the loop
                asm volatile("" : "+v"(voff), "+s"(blk), "+s"(half), "+s"(dst), "+s"(dhalf));
                vm_dma16(src, voff + (uint32_t)qb * blk + (uint32_t)i * half, dst + (uint32_t)(slot * kLandE * (int)sizeof(E)) + (uint32_t)i * dhalf);
            }
        } else if (wave < 3) {
            const int ln = lane_now();
            const int dc = (ln & 3) * 8;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int r = min(32 * qb + 16 * i + (ln >> 2), N - 1);
                vm_dma16(src, row_byte_offset<E>(unit_row<MAPPED>(p.map, b, r), mine_sn, dc), lds_addr(&lds_raw[slot][wave * 1024 + 16 * i * 32]));
            }
        } else {
            const int ln = lane_now();
            const int r = min(32 * qb + (ln & 31), N - 1);
            vm_dma4(src, 4u * (uint32_t)r, lds_addr(&lds_raw[slot][3 * 1024]));
            vm_dma4(src, 4u * (uint32_t)r, lds_addr(&lds_raw[slot][3 * 1024]));
        }
    };

    // ---- landing slot -> tile slot: q_hat * s * log2e, dO, -delta, -lse * log2e, 1 / |q|.  Thread = 4 columns of one
    // row (8 threads per row, 32 rows; wavefront w has rows 8 w .. 8 w + 7).  Straight-line code: of the eight lanes
    // of a row, lane 0 writes -delta, lane 1 -lse * log2e, lane 2 1 / |q| and the rest a word nobody reads, through one
    // store whose address and value are selected per lane.  In two halves, so that the reads of all the side
    // stages of an iteration can be issued before anything waits for one of them. ----
    struct NormIn { V4 q4, do4, o4; float lse; };
    auto normalise_load = [&](int lslot) __attribute__((always_inline)) -> NormIn {
        const int r = tid >> 3, c4 = (tid & 7) * 4;
        NormIn x;
        x.q4 = *reinterpret_cast<const V4*>(&lds_raw[lslot][0 * 1024 + r * 32 + c4]);
        x.do4 = *reinterpret_cast<const V4*>(&lds_raw[lslot][1 * 1024 + r * 32 + c4]);
        x.o4 = *reinterpret_cast<const V4*>(&lds_raw[lslot][2 * 1024 + r * 32 + c4]);
        x.lse = reinterpret_cast<const float*>(&lds_raw[lslot][3 * 1024])[r];
        return x;
    };
    auto normalise_store = [&](NormIn x, int qb, int tslot) __attribute__((always_inline)) {
        const int r = tid >> 3, c4 = (tid & 7) * 4;
        const int row = 32 * qb + r;
        if (!PLAIN && row >= N) {
#pragma unroll
            for (int j = 0; j < 4; j++) { x.q4[j] = 0; x.do4[j] = 0; }
        }
        const float sq = oct_add(dot4(x.q4, x.q4));
        const float dl = oct_add(dot4(x.o4, x.do4));
        const float inv = inv_norm_fast(sq);
        const float iq = inv * scale2;
        SV4 qn;
#pragma unroll
        for (int j = 0; j < 4; j++) qn[j] = (SE)((float)x.q4[j] * iq);
        *reinterpret_cast<SV4*>(&lds_Qs[tslot][r * kRow + c4]) = qn;
        *reinterpret_cast<V4*>(&lds_dOs[tslot][r * kRow + c4]) = x.do4;
        const float l2 = ((PLAIN || row < N) && x.lse != -INFINITY) ? -x.lse * kLog2e : -INFINITY;   // padded / fully masked rows: P = 0
        const int role = tid & 7;
        (&lds_meta[tslot][0][0])[meta_lane] = role == 0 ? -dl : role == 1 ? l2 : inv;
    };
    auto normalise = [&](int qb, int lslot, int tslot) __attribute__((always_inline)) {
        normalise_store(normalise_load(lslot), qb, tslot);
    };

    // ---- dq of block qb of unit b: sum of the four wavefronts' partials, back through q / max(|q|, eps); wavefront w
    // takes rows 8 w .. 8 w + 7 (the rows it normalised: it may read them from a tile slot right before it
    // overwrites that slot), lane = 4 columns of one row.  q_hat is taken back from the score operand. ----
    float ds_acc = 0.f;
    const char* const dq_base = reinterpret_cast<const char*>(p.dq.ptr) + (int64_t)h * p.dq.sh * (int64_t)sizeof(E);
    struct SumIn { f32x4 part[WAVES]; SV4 qs; float inv; };
    auto sum_load = [&](int pslot, int tslot) __attribute__((always_inline)) -> SumIn {
        const int r = tid >> 3, c4 = (tid & 7) * 4;
        SumIn x;
#pragma unroll
        for (int w = 0; w < WAVES; w++) x.part[w] = *reinterpret_cast<const f32x4*>(&lds_part[pslot][w][r * kPartRow + c4]);
        x.qs = *reinterpret_cast<const SV4*>(&lds_Qs[tslot][r * kRow + c4]);
        x.inv = lds_meta[tslot][2][r];
        return x;
    };
    const uint32_t dq_lane = (uint32_t)(((tid >> 3) * (int)p.dq.sn + (tid & 7) * 4) * (int)sizeof(E));
    const uint32_t dq_rows32 = (uint32_t)(32 * (int)p.dq.sn * (int)sizeof(E));
    auto sum_store = [&](const SumIn& x, const char* dq_unit, int b, int qb) __attribute__((always_inline)) {
        const int ln = lane_now();
        const int r = 8 * wave + (ln >> 3), c4 = (ln & 7) * 4;
        f32x4 acc = x.part[0];
#pragma unroll
        for (int w = 1; w < WAVES; w++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += x.part[w][j];
        // with qs = q_hat s2 (s2 = s log2e):  dq = s / |q| (acc - q_hat (q_hat . acc)) = f acc - qs (f (qs . acc) / s2^2)
        float dots = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) dots += acc[j] * (float)x.qs[j];
        dots = oct_add(dots);
        const float dot = dots * unscale;                               // q_hat . dq_hat / s: the row's dlogit_scale term
        const float f = s_true * x.inv;
        const float c = x.inv < 0.5f / kNormEps ? f * dot * unscale : 0.f;      // |q| <= eps: no projection
        V4 o4;
#pragma unroll
        for (int j = 0; j < 4; j++) o4[j] = (E)(f * acc[j] - (float)x.qs[j] * c);
        const int q = 32 * qb + r;
        if (PLAIN) {
            uint32_t voff = dq_lane;
            asm volatile("" : "+v"(voff));
            vm_store8(const_cast<char*>(dq_unit), voff + (uint32_t)qb * dq_rows32, o4);
            ds_acc += (ln & 7) == 0 ? dot : 0.f;
        } else {
            const int qrow = min(q, N - 1);
            E* dst = reinterpret_cast<E*>(const_cast<char*>(dq_unit) + row_byte_offset<E>(unit_row<MAPPED>(p.map, b, qrow), p.dq.sn, c4));
            vm_store8_if_below(dst, o4, q, N);
            ds_acc += ((ln & 7) == 0 && q < N) ? dot : 0.f;
        }
    };
    auto sum_block = [&](int b, int qb, int pslot, int tslot) __attribute__((always_inline)) {
        sum_store(sum_load(pslot, tslot), unit_start(dq_base, p.dq.sb, b), b, qb);
    };

    // The rows of the wavefront's own keys (k and v, 16 bytes per lane and key tile) skip the landing area: they
    // are requested after the last block of a unit and used once the dk / dv of that unit have been stored.
    V8 kraw[KT], vraw[KT];
    // byte offset of this lane's 16 bytes of key row 64 wave + l16 in a tensor with rows `sn` elements apart (whole
    // windows without a map: the other key tiles are 16 rows further on each)
    auto key_lane_offset = [&](int64_t sn) -> uint32_t {
        const int ln = lane_now();
        return (uint32_t)(((64 * wave + (ln & 15)) * (int)sn + 8 * (ln >> 4)) * (int)sizeof(E));
    };
    auto fetch_keys = [&](int b) __attribute__((always_inline)) {
        if (PLAIN) {
            const char* ku = unit_start(reinterpret_cast<const char*>(p.k.ptr) + (int64_t)h * p.k.sh * (int64_t)sizeof(E), p.k.sb, b);
            const char* vu = unit_start(reinterpret_cast<const char*>(p.v.ptr) + (int64_t)h * p.v.sh * (int64_t)sizeof(E), p.v.sb, b);
            const uint32_t ko = key_lane_offset(p.k.sn), vo = key_lane_offset(p.v.sn);
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
                kraw[kt] = ld8<V8>(reinterpret_cast<const E*>(ku + (ko + (uint32_t)(16 * kt * (int)sizeof(E)) * (uint32_t)p.k.sn)));
                vraw[kt] = ld8<V8>(reinterpret_cast<const E*>(vu + (vo + (uint32_t)(16 * kt * (int)sizeof(E)) * (uint32_t)p.v.sn)));
            }
            return;
        }
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

    // ---- fill the pipeline: blocks 0 and 1 of the first unit as tiles, block 2 in its landing slot ----
    const bool any = cur.t < t_end;
    if (any) {
        if (HAS_TAB) {
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int tt = 0; tt < 2; tt++) tb[kt][tt] = *reinterpret_cast<const f32x4*>(cur.tab + lane4 + (((kt * NQB) * 2 + tt) << 8));
        }
        dma_block(source_of(cur.b), cur.b, 0, 0);
        dma_block(source_of(cur.b), cur.b, 1, 1);
        fetch_keys(cur.b);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    if (any) {
        normalise(0, 0, 0);
        normalise(1, 1, 1);
    }
    __syncthreads();
    if (any) {
        dma_block(source_of(cur.b), cur.b, 2, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();

    bool have_prev = false;      // a block whose dq partials wait for their sum
    int b_prev = 0;
    const char* dq_prev = nullptr;
    // lane parts of the LDS addresses inside a tile slot; what depends on the block is a compile-time constant
    const int row_base = (8 * (l16 >> 2) + (l16 & 3)) * kRow + 8 * g;       // + 4 t * kRow
    const int tr_base = (8 * g + (l16 >> 2)) * kRow + 8 * (l16 & 3);         // + 4 dt (+ 4 kRow)
    SE* const zst = &lds_zst[0][0] + wave * (64 * kRow);

    // ---- dQ_hat^T of a block over this wavefront's keys: B operand = dZ^T out of the slab, A operand = K_hat^T.
    // Column n of query tile t is query 8 (n / 4) + 4 t + n % 4 of the block; the lane's rows are d = 8 g + 4 dt + i.
    // The partial goes to LDS as [query][d]. ----
    SV8 akt[2][2];
    auto dq_load = [&](SV8 (&bz)[2][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int t = 0; t < 2; t++)
                bz[c][t] = lds_tr8<SDT>(zst + 32 * c * kRow + tr_base + 4 * t, zst + 32 * c * kRow + tr_base + 4 * t + 4 * kRow);
    };
    auto dq_products = [&](const SV8 (&bz)[2][2], int pslot) __attribute__((always_inline)) {
        f32x4 dqa[2][2];
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) dqa[dt][t][i] = 0.f;
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int dt = 0; dt < 2; dt++) dqa[dt][t] = Elem<SDT>::mfma16(akt[dt][c], bz[c][t], dqa[dt][t]);
        float* part = &lds_part[pslot][0][0] + wave * (32 * kPartRow);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
                *reinterpret_cast<f32x4*>(part + (8 * (l16 >> 2) + 4 * t + (l16 & 3)) * kPartRow + 8 * g + 4 * dt) = dqa[dt][t];
    };

    while (cur.t < t_end) {
        const int b = cur.b;
        const bool have_next = nxt.t < t_end;
        // without a next unit the read-ahead fetches this one again: harmless, and the loop body stays free of branches
        const int b_next = have_next ? nxt.b : b;
        const float* tab = cur.tab;
        const float* tab_next = have_next ? nxt.tab : tab;
        Unit after = nxt;
        const char* const src_cur = source_of(b);
        const char* const src_next = source_of(b_next);
        const char* const dq_cur = unit_start(dq_base, p.dq.sb, b);

        // ---- this wavefront's keys: k_hat (score type) and v as B operands, 1 / |k| for the epilogue ----
        SV8 bk[KT];
        V8 bv[KT];
        float kinv[KT];     // negative: |k| <= eps, the projection term of the Jacobian is dropped
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int key = 64 * wave + 16 * kt + l16;
            V8 k8 = kraw[kt];
            bv[kt] = vraw[kt];
            if (!PLAIN && key >= N) { k8 = zero8<V8>(); bv[kt] = zero8<V8>(); }
            const float sk = col_add(dot8(k8, k8));
            const float ik = inv_norm_fast(sk);
#pragma unroll
            for (int j = 0; j < 8; j++) bk[kt][j] = (SE)((float)k8[j] * ik);
            kinv[kt] = sk > kNormEps * kNormEps ? ik : -ik;
        }
        // K_hat^T of the same keys as the A operand of dQ_hat^T += K_hat^T dZ^T: through the wavefront's own slab.
        // A row m <-> d = 8 (m / 4) + 4 dt + m % 4; k-slots 8 g + j <-> key 32 c + 8 g + j of the wavefront.
#pragma unroll
        for (int kt = 0; kt < KT; kt++) st8<SV8>(zst + (16 * kt + l16) * kRow + 8 * g, bk[kt]);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int c = 0; c < 2; c++)
                akt[dt][c] = lds_tr8<SDT>(zst + 32 * c * kRow + tr_base + 4 * dt, zst + 32 * c * kRow + tr_base + 4 * dt + 4 * kRow);
        asm volatile("" ::: "memory");

        f32x4 dvacc[KT][2], dkacc[KT][2];
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
#pragma unroll
                for (int i = 0; i < 4; i++) { dvacc[kt][dt][i] = 0.f; dkacc[kt][dt][i] = 0.f; }

        // LDS operands of a block.  The rows of Q_hat and dO and -delta are only read by the S and dP products, so
        // their registers are refilled with the coming block's values as soon as the last such product of a block
        // has been issued (the coming block's tiles were written an iteration ago); -lse and the transposed
        // operands are read at the top of their block and arrive behind the first products.
        SV8 aq[2];
        V8 ado[2];
        f32x4 nd[2];
        auto load_rows = [&](int qb) __attribute__((always_inline)) {
            const int s = qb & 3;
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                aq[tt] = ld8<SV8>(&lds_Qs[s][row_base + 4 * tt * kRow]);
                ado[tt] = ld8<V8>(&lds_dOs[s][row_base + 4 * tt * kRow]);
                nd[tt] = *reinterpret_cast<const f32x4*>(&lds_meta[s][0][8 * g + 4 * tt]);
            }
        };
        load_rows(0);
        SV8 bz[2][2];      // dZ^T of the block before: read behind its last key tile, used at the top of the next iteration

#pragma unroll
        for (int qb = 0; qb < NQB; qb++) {
            // ---- the other stages of the pipeline, all independent of each other: their LDS reads first, then the
            // arithmetic (the dq products run on the matrix pipe meanwhile), the stores to memory last ----
            {
                const bool do_dq = qb > 0;                 // block 7's products follow the loop
                const bool do_sum = qb >= 2 || have_prev;
                SumIn si;
                if (do_sum) si = sum_load(qb & 1, (qb + 2) & 3);
                const NormIn ni = normalise_load(qb & 1);
                dma_block(qb + 3 < NQB ? src_cur : src_next, qb + 3 < NQB ? b : b_next, (qb + 3) & 7, (qb + 3) & 1);
                if (do_dq) dq_products(bz, (qb - 1) & 1);
                if (do_sum) sum_store(si, qb >= 2 ? dq_cur : dq_prev, qb >= 2 ? b : b_prev, (qb + 6) & 7);
                normalise_store(ni, (qb + 2) & 7, (qb + 2) & 3);
            }
            __builtin_amdgcn_sched_barrier(0);

            // ---- block qb against the wavefront's 64 keys ----
            const int s = qb & 3;
            f32x4 nl[2];
            V8 tdo[2];
            SV8 tq[2];
#pragma unroll
            for (int tt = 0; tt < 2; tt++) nl[tt] = *reinterpret_cast<const f32x4*>(&lds_meta[s][1][8 * g + 4 * tt]);
#pragma unroll
            for (int dt = 0; dt < 2; dt++) {
                // A row m <-> d = 8 (m / 4) + 4 dt + m % 4: the lane's dk / dv values are d = 8 g + 4 dt + i
                tdo[dt] = lds_tr8<DT>(&lds_dOs[s][tr_base + 4 * dt], &lds_dOs[s][tr_base + 4 * dt + 4 * kRow]);
                tq[dt] = lds_tr8<SDT>(&lds_Qs[s][tr_base + 4 * dt], &lds_Qs[s][tr_base + 4 * dt + 4 * kRow]);
            }
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
                f32x4 sacc[2], pacc[2];
                // (The table values of this key tile were requested a block ago by ordinary loads, which the compiler
                // waits for by count.  They must stay ordinary loads: a load hidden in inline assembly delivers into
                // registers the compiler believes written already, and it is free to move such a value elsewhere
                // -- into an accumulator register, say -- before the data has arrived.)
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
                if (kt == KT - 1) load_rows((qb + 1) & 7);
                // the dbias accumulators of the last blocks come out of LDS: requested here, used behind the exponentials
                f32x4 dbs[2];
                if (HAS_BIAS && db_in_lds(qb)) {
#pragma unroll
                    for (int hf = 0; hf < 2; hf++)
                        dbs[hf] = *reinterpret_cast<const f32x4*>(lds_db + ((((qb - (NQB - kLdsQb)) * KT + kt) * 2 + hf) * NT + tid) * 4);
                }
                // everything read ahead is on its way before this tile's elementwise work starts
                asm volatile("" : "+v"(sacc[0]), "+v"(sacc[1]) :: "memory");
                if (kt == 2 && qb == 3 && have_next) after = unit_at(nxt.t + p.groups);      // scalar work, off the critical path
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
                // dZ of this key tile, [key][query], for the transposed read below
                st8<SV8>(zst + (16 * kt + l16) * kRow + 8 * g, z8);
                if (HAS_BIAS) {
#pragma unroll
                    for (int hf = 0; hf < 2; hf++) {
                        if (db_in_lds(qb)) {
                            f32x4* slot = reinterpret_cast<f32x4*>(lds_db + ((((qb - (NQB - kLdsQb)) * KT + kt) * 2 + hf) * NT + tid) * 4);
                            *slot = Elem<SDT>::mfma16(sel[hf], z8, dbs[hf]);
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
            // dZ^T of this block for the dq products of the next iteration: the wavefront's own data, so the reads
            // need not wait for the barrier, and the barrier need not wait for them: it waits until the 8 youngest
            // LDS operations (these reads) are all that is outstanding, i.e. for every write before them.
            asm volatile("" ::: "memory");
            dq_load(bz);
            // The rows requested at the top of this iteration are tiles in the next one: they have landed once at most
            // the table loads issued since (8) are outstanding.
            if (HAS_TAB) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            asm volatile("s_waitcnt lgkmcnt(8)\n\ts_barrier" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
        dq_products(bz, 1);       // block 7; its sum follows in the second iteration from here (or behind the loop)
        asm volatile("" ::: "memory");
        fetch_keys(b_next);
        // ---- epilogue dk, dv: lane (key, g) holds d = 8 g + 4 dt + i, which is 16 bytes of a row ----
        const int ln_e = lane_now();
        const char* dk_unit = nullptr;
        const char* dv_unit = nullptr;
        uint32_t dk_off = 0, dv_off = 0;
        if (PLAIN) {
            dk_unit = unit_start(reinterpret_cast<const char*>(p.dk.ptr) + (int64_t)h * p.dk.sh * (int64_t)sizeof(E), p.dk.sb, b);
            dv_unit = unit_start(reinterpret_cast<const char*>(p.dv.ptr) + (int64_t)h * p.dv.sh * (int64_t)sizeof(E), p.dv.sb, b);
            dk_off = key_lane_offset(p.dk.sn);
            dv_off = key_lane_offset(p.dv.sn);
        }
#pragma unroll
        for (int kt = 0; kt < KT; kt++) {
            const int l16 = ln_e & 15, g = ln_e >> 4;
            const int key = 64 * wave + 16 * kt + l16;
            // dk = (dk_hat - k_hat (k_hat . dk_hat)) / |k| with dk_hat = ln2 * accumulator (undoing the log2e folded into Q_hat)
            float x[8];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                x[j] = (float)bk[kt][j];
                dot += dkacc[kt][j >> 2][j & 3] * x[j];
            }
            dot = col_add(dot);
            const float c = fabsf(kinv[kt]) * kLn2;
            const float proj = kinv[kt] > 0.f ? dot : 0.f;
            V8 o8, v8;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                o8[j] = (E)(c * (dkacc[kt][j >> 2][j & 3] - x[j] * proj));
                v8[j] = (E)dvacc[kt][j >> 2][j & 3];
            }
            if (PLAIN) {
                vm_store16(const_cast<char*>(dk_unit), dk_off + (uint32_t)(16 * kt * (int)sizeof(E)) * (uint32_t)p.dk.sn, o8);
                vm_store16(const_cast<char*>(dv_unit), dv_off + (uint32_t)(16 * kt * (int)sizeof(E)) * (uint32_t)p.dv.sn, v8);
            } else {
                // keys beyond n (only with n < 256) address row n - 1 and are masked out of the store
                const int krow = min(key, N - 1);
                vm_store16_if_below(const_cast<E*>(row_ptr<MAPPED, E>(p.dk, p.map, b, h, krow)) + 8 * g, o8, key, N);
                vm_store16_if_below(const_cast<E*>(row_ptr<MAPPED, E>(p.dv, p.map, b, h, krow)) + 8 * g, v8, key, N);
            }
        }
        b_prev = b;
        dq_prev = dq_cur;
        have_prev = true;
        cur = nxt;
        nxt = after;
    }
    // the last two blocks of the last unit
    if (have_prev) {
        lds_barrier();
        sum_block(b_prev, NQB - 2, 0, 2);
        sum_block(b_prev, NQB - 1, 1, 3);
    }

    // ---- dlogit_scale: one partial per workgroup ----
    if (p.scale_kind == FWA2_SCALE_TENSOR) {
        const float wsum = wave_sum(ds_acc);
        if (lane == 0) lds_red[wave] = wsum;
        __syncthreads();
        if (tid == 0) {
            float tot = 0.f;
#pragma unroll
            for (int i = 0; i < WAVES; i++) tot += lds_red[i];
            p.part_dscale[(int64_t)h * p.ds_parts + grp] = tot * s_true;
        }
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
                    // (a plain store: the reduction that follows then finds the tiles in the memory-side cache)
                    *reinterpret_cast<f32x4*>(dst + 32 * qb + 16 * hf + 4 * g) = acc;
                }
        }
    }
}

// ---- host side -----------------------------------------------------------------
template <int DT, bool HAS_BIAS, bool HAS_TAB, bool MASKED, int ROWS>
static hipError_t launch_one(BwdParams p, hipStream_t st, int max_groups, int* groups_out) {
    static std::atomic<int> fit_by_device[kFitDevices];
    const int fit = resident_per_cu_cached(bwd_one_kernel<DT, HAS_BIAS, HAS_TAB, MASKED, ROWS>, one256::NT, fit_by_device);
    int groups = (p.cus * fit) / p.heads;
    if (groups < 1) groups = 1;
    if (groups > max_groups) groups = max_groups;
    p.groups = groups;
    p.db_parts = groups;
    p.db_slot0 = 0;
    p.ds_parts = groups;
    hipLaunchKernelGGL((bwd_one_kernel<DT, HAS_BIAS, HAS_TAB, MASKED, ROWS>), dim3(p.heads * groups), dim3(one256::NT), 0, st, p);
    if (groups_out) { groups_out[0] = groups; groups_out[1] = groups; }
    return hipGetLastError();
}

template <int DT>
static hipError_t launch_one_dt(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out) {
    const bool masked = mask_dt >= 0;
    const bool has_tab = has_bias || masked || p.n < one256::R;
    const bool mapped = p.map.nw > 0;
    hipError_t e = launch_score_tables(p, DT, has_bias, mask_dt, st);
    if (e != hipSuccess) return e;
    if (p.ev_start) (void)hipEventRecord(p.ev_start, st);
#define FWA2_ONE_CASE(B, T, M)                                                                                       \
    (mapped ? launch_one<DT, B, T, M, 1>(p, st, max_groups, groups_out)                                              \
            : p.n == one256::R ? launch_one<DT, B, T, M, 2>(p, st, max_groups, groups_out) : launch_one<DT, B, T, M, 0>(p, st, max_groups, groups_out))
    if (has_bias) e = masked ? FWA2_ONE_CASE(true, true, true) : FWA2_ONE_CASE(true, true, false);
    else if (masked) e = FWA2_ONE_CASE(false, true, true);
    else if (has_tab) e = FWA2_ONE_CASE(false, true, false);
    else e = mapped ? launch_one<DT, false, false, false, 1>(p, st, max_groups, groups_out)
                    : launch_one<DT, false, false, false, 2>(p, st, max_groups, groups_out);      // no table: 256 tokens
#undef FWA2_ONE_CASE
    if (p.ev_stop) (void)hipEventRecord(p.ev_stop, st);
    return e;
}

#if FWA2_HALF == 2
hipError_t launch_backward_one_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out) {
    return launch_one_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, groups_out);
}
#else
#if FWA2_HALF == 1
hipError_t launch_backward_one_f16(const BwdParams& p, bool has_bias, int mask_dt, hipStream_t st, int max_groups, int* groups_out);
#endif
// dq, dk, dv, the dbias partial tiles and the dscale partials of a call with 161 .. 256 tokens per window; p.tab
// points at room for heads * (1 + windows) tables of 256 x 256 floats.  groups_out: workgroups per head (= dscale
// partials per head), dbias partial tiles per head.
hipError_t launch_backward_one(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st, int max_groups,
                               int* groups_out) {
    if (dtype == FWA2_BF16) return launch_one_dt<FWA2_BF16>(p, has_bias, mask_dt, st, max_groups, groups_out);
#if FWA2_HALF == 1
    return launch_backward_one_f16(p, has_bias, mask_dt, st, max_groups, groups_out);
#else
    return launch_one_dt<FWA2_F16>(p, has_bias, mask_dt, st, max_groups, groups_out);
#endif
}
#endif

}  // namespace fwa2
