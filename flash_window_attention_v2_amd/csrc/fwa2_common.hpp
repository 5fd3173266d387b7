// Shared device helpers for the gfx950 window-attention kernels: vector types,
// MFMA wrappers for bf16 / fp16, cross-lane reductions on 64-wide wavefronts,
// LDS transpose reads and the launch-side parameter block.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/fwa2.h"

namespace fwa2 {

// Workgroups of `kern` that fit on one compute unit of the CURRENT device: asked from the runtime once per device
// and call site (`slots` is the call site's static array, kFitDevices entries; a benign race at worst repeats
// the query).  Persistent workgroups should all be resident at once: one that waits for a slot starts its share
// late (nothing depends on it for correctness).
constexpr int kFitDevices = 64;
template <class K>
static inline int resident_per_cu_cached(K kern, int threads, std::atomic<int>* slots) {
    int dev = 0;
    const bool tracked = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kFitDevices;
    int n = tracked ? slots[dev].load(std::memory_order_relaxed) : 0;
    if (n == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, threads, 0) != hipSuccess || n < 1) n = 1;
        if (tracked) slots[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kLn100 = 4.605170185988092f;
constexpr float kNormEps = 1e-12f;
constexpr int kScoreDT = FWA2_F16;   // element type of q_hat / k_hat in the forward score product

// Element-type traits: E = storage element, V8 / V4 = 8- and 4-wide vectors.
template <int DT> struct Elem;
template <> struct Elem<FWA2_BF16> {
    typedef __bf16 E;
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ V4 lds_tr(const E* p) {
        return __builtin_bit_cast(V4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                          (__attribute__((address_space(3))) s16x4*)(p)));
    }
};
template <> struct Elem<FWA2_F16> {
    typedef _Float16 E;
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ V4 lds_tr(const E* p) {
        return __builtin_bit_cast(V4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                          (__attribute__((address_space(3))) s16x4*)(p)));
    }
};

// 16-byte global / LDS accesses of 8 elements.
template <class V8, class E>
__device__ __forceinline__ V8 ld8(const E* p) { return *reinterpret_cast<const V8*>(p); }
template <class V8, class E>
__device__ __forceinline__ void st8(E* p, V8 v) { *reinterpret_cast<V8*>(p) = v; }

// 16-byte store of an output row chunk that nobody re-reads soon: non-temporal, like the row fetches.  (STREAM =
// false: a plain store, for kernels whose whole problem fits the memory-side cache often enough that the next
// kernel finds the rows there.)
template <class V8, class E, bool STREAM = true>
__device__ __forceinline__ void st8_stream(E* p, V8 v) {
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<V8*>(p));
    else *reinterpret_cast<V8*>(p) = v;
}

template <class V8>
__device__ __forceinline__ V8 zero8() {
    V8 z;
#pragma unroll
    for (int j = 0; j < 8; j++) z[j] = 0;
    return z;
}

// An LDS array that every function instantiated with the same arguments shares: the two bodies a kernel may run
// (one per class of windows) name the same arrays this way, so the kernel's LDS is that of one body.
template <class T, int COUNT, int TAG>
__device__ __forceinline__ __attribute__((returns_nonnull)) T* shared_array() {
    __shared__ __attribute__((aligned(16))) T a[COUNT];
    return a;
}

// Sum of the squares of 8 packed elements on the dot unit (two products per instruction, fp32 accumulation).
__device__ __forceinline__ float sumsq8(bf16x8 a) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v2 x;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1];
        s = __builtin_amdgcn_fdot2_f32_bf16(x, x, s, false);
    }
    return s;
}
__device__ __forceinline__ float sumsq8(f16x8 a) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v2 x;
        x[0] = a[2 * j]; x[1] = a[2 * j + 1];
        s = __builtin_amdgcn_fdot2(x, x, s, false);
    }
    return s;
}

// Two transposing LDS reads glued into one 8-element MFMA operand.
template <int DT>
__device__ __forceinline__ typename Elem<DT>::V8 lds_tr8(const typename Elem<DT>::E* lo,
                                                         const typename Elem<DT>::E* hi) {
    typename Elem<DT>::V4 a = Elem<DT>::lds_tr(lo);
    typename Elem<DT>::V4 b = Elem<DT>::lds_tr(hi);
    typename Elem<DT>::V8 r;
#pragma unroll
    for (int j = 0; j < 4; j++) { r[j] = a[j]; r[4 + j] = b[j]; }
    return r;
}

// ---- global -> LDS copies that bypass the registers, issued by hand ---------------------------------------
// The builtin form of these loads makes the compiler guard LDS reads it cannot tell apart from the landing area
// with a wait for ALL outstanding vector-memory operations, which stalls a kernel that fetches the next unit while
// it computes on the current one.  Written as inline assembly the copies are invisible to that bookkeeping: the
// kernel waits for them itself (s_waitcnt vmcnt) before it reads a landing area.  Each lane reads 16 (or 4) bytes
// at its own address; lane i lands at lds + 16 i (4 i), lds being uniform over the wavefront.  The waits the
// hardware asks for around M0 are part of the sequence.
__device__ __forceinline__ uint32_t lds_address(const void* p) {     // of a wavefront-uniform pointer, as a scalar
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p);
}
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16_to_lds(const void* src, uint32_t lds) {      // non-temporal: streamed rows
    asm volatile("s_nop 3\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(src), "s"(lds) : "memory", "m0");
}
// The same from a wavefront-uniform base (scalar registers) plus a 32-bit byte offset per lane: no 64-bit
// address arithmetic on the vector unit.
__device__ __forceinline__ const void* uniform_pointer(const void* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const void*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void dma16_to_lds(const void* uniform_base, uint32_t byte_offset, uint32_t lds) {
    asm volatile("s_nop 3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(byte_offset), "s"(uniform_base), "s"(lds) : "memory", "m0");
}
// Byte offset of (row, col) inside a unit whose rows are `sn` elements apart (one 24-bit multiply).
template <class E>
__device__ __forceinline__ uint32_t row_byte_offset(int row, int64_t sn, int col) {
    uint32_t prod;
    asm("v_mul_u32_u24 %0, %1, %2" : "=v"(prod) : "s"((uint32_t)sn), "v"((uint32_t)row));
    return (prod + (uint32_t)col) * (uint32_t)sizeof(E);
}
__device__ __forceinline__ void dma4_to_lds(const void* src, uint32_t lds) {
    asm volatile("s_nop 3\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
}
#pragma clang diagnostic pop

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global store the
// wavefront has issued (it fences global memory at workgroup scope); in a loop that ends with output stores
// that puts a full write round trip on the critical path of every iteration, with all wavefronts parked at
// the barrier.  The kernels that use this exchange data through LDS alone.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Issue priority that falls as a wavefront advances through the `steps` key groups of a unit (3 in the first
// quarter ... 0 in the last and in everything up to the next unit's first group).  The arbiter otherwise favours the
// oldest wavefront of a SIMD, which then reaches the barrier early and leaves the end of every unit to one
// wavefront per SIMD with nothing to hide its waits; with this, whoever is behind goes first and the wavefronts
// of a SIMD finish together.
__device__ __forceinline__ void progress_priority(int step, int steps) {
    if (steps < 4) return;
    if (step == 0) __builtin_amdgcn_s_setprio(3);
    else if (step == steps / 4) __builtin_amdgcn_s_setprio(2);
    else if (step == steps / 2) __builtin_amdgcn_s_setprio(1);
    else if (step == 3 * steps / 4) __builtin_amdgcn_s_setprio(0);
}

// ---- cross-lane helpers (wave64) -------------------------------------------
// Value held by the lane 32 away, combined with the own value by max / add.
__device__ __forceinline__ float xor32_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_add(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_add(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Sum over the 4 lanes of an aligned quad (DPP quad_perm, no LDS traffic).
__device__ __forceinline__ float quad_add(float x) {
    float y = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0xB1, 0xF, 0xF, true));
    x += y;   // lanes (0,1) (2,3) paired
    y = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x4E, 0xF, 0xF, true));
    return x + y;
}

// Lane index recomputed on the spot (two VALU instructions, never hoisted): what is derived from it
// need not stay in a register, or in scratch, across the phases of a unit.
__device__ __forceinline__ int lane_now() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// 1 / max(||x||, eps) from a sum of squares (torch.nn.functional.normalize): one v_rsq_f32 (1 ulp) instead of
// a square root and an IEEE division (about twenty instructions); every use is rounded to 16 bits afterwards.
__device__ __forceinline__ float inv_norm(float sumsq) {
    return __builtin_amdgcn_rsqf(fmaxf(sumsq, kNormEps * kNormEps));
}

// Row r of a 32-row MFMA A operand <-> position inside a 32-key tile such that
// the 8 accumulator registers a lane feeds to the next MFMA as its k-slots are
// 8 consecutive positions: swap bits 2 and 3 of r.
__host__ __device__ constexpr int swap_bits23(int r) {
    return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1);
}


// ---- small shared device helpers ------------------------------------------------
template <class V8>
__device__ __forceinline__ void unpack8(V8 v, float* x) {
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = (float)v[j];
}

// 8 consecutive elements starting at column c0 of one row of bias / mask, as floats.
// VEC: the row may be read with 16-byte loads and n is a multiple of 8; columns at or
// beyond n are then read from the last 8 real columns instead (the caller overwrites the
// scores of such padded keys with -inf), which keeps the load in bounds without a branch.
// !VEC: element loads with a bounds check, padded columns read as 0.
template <bool VEC, class E>
__device__ __forceinline__ void load_row8(const E* row, int c0, int n, float* x) {
    typedef E V8 __attribute__((ext_vector_type(8)));
    if (VEC) {
        const V8 v = *reinterpret_cast<const V8*>(row + min(c0, n - 8));
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = (float)v[j];
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = (c0 + j < n) ? (float)row[c0 + j] : 0.f;
    }
}

// Element type of the mask: the input dtype, or float for an fp32 mask.
template <int DT, int MASK_DT> struct MaskElem { typedef typename Elem<DT>::E E; };
template <int DT> struct MaskElem<DT, FWA2_F32> { typedef float E; };

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
    return x;
}

// ---- helpers of the kernels that keep the bias tile resident in registers ----
constexpr int kLiveCache = 1024;    // windows whose mask flags are cached in LDS
constexpr float kGapLimit = 96.f;   // largest tolerated (row bound - largest logit), log2 domain

// A window whose mask is exactly value * [id_i != id_j] (see mask_scan_kernel) is described by this record
// instead of its N x N entries.  The kernels add the term on the matrix pipe: one more (small) MFMA per score
// tile whose query-side operand holds value * log2e, split into two fp16 terms, in the k-slot of the query's
// id, and whose key-side operand holds 1 in every slot but the key's own id.
constexpr int kMaxRegions = 8;
constexpr float kMaxRegionValue2 = 30000.f;     // |value * log2e| must stay inside fp16 with room to spare
struct RegionRecord {
    float value;
    int count;
    int pad[2];
    uint8_t id[256];
};
static_assert(sizeof(RegionRecord) == 272, "RegionRecord is part of the C ABI (FWA2_MASK_REGION_BYTES)");
// The region product is a 16 x 16 x 16 fp16 MFMA whose 16 k-slots are (8 ids) x (value * log2e split into two
// fp16 terms).  Lane (g, l16) of an operand holds slots 4g .. 4g+3: ids 4 (g & 1) .. 4 (g & 1) + 3, first term for
// g < 2, second term for g >= 2.  `key_side` is the M operand (rows = keys), `query_side` the N operand.
__device__ __forceinline__ f32x4 region_mfma(f16x4 key_side, f16x4 query_side, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(key_side, query_side, c, 0, 0, 0);
}
// Query-side operand of this lane for a query with region id `id`: value2 = value * log2e.
__device__ __forceinline__ f16x4 region_query_operand(float value2, int id, int g) {
    const _Float16 hi = (_Float16)value2;
    const _Float16 lo = (_Float16)(value2 - (float)hi);
    const _Float16 term = g < 2 ? hi : lo;
    const int rel = id - 4 * (g & 1);
    f16x4 r;
#pragma unroll
    for (int j = 0; j < 4; j++) r[j] = j == rel ? term : (_Float16)0.f;
    return r;
}
// Key-side table entry of a key with region id `id`: 1 in every id slot but its own (8 halves, ids 0 .. 7); a lane
// reads the four halves at 4 (g & 1).
__device__ __forceinline__ f16x8 region_key_entry(int id) {
    f16x8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = j == id ? (_Float16)0.f : (_Float16)1.f;
    return r;
}

__device__ __forceinline__ float xor16_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// reductions over the 4 lanes (g = 0..3) that share a query column
__device__ __forceinline__ float col_max(float x) { return xor32_max(xor16_max(x)); }
__device__ __forceinline__ float col_add(float x) { return xor32_add(xor16_add(x)); }

// 8 consecutive entries of a bias / mask row in their storage type; columns >= n read as `pad`.
template <bool VEC, class T>
__device__ __forceinline__ auto load_raw8(const T* row, int c0, int n, float pad) {
    typedef T TV8 __attribute__((ext_vector_type(8)));
    TV8 v;
    if (VEC) {   // rows 16-byte aligned and at least n rounded up to 8 entries long: a whole group can be read
        if (c0 < n) {
            v = *reinterpret_cast<const TV8*>(row + c0);
            if (c0 + 8 > n) {   // the last group of a row whose length is not a multiple of 8: the tail is padding
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = (c0 + i < n) ? v[i] : (T)pad;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = (T)pad;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (c0 + i < n) ? row[c0 + i] : (T)pad;
    }
    return v;
}

// Cache policy of the streaming q / k / v / dO / o row fetches: non-temporal, so that rows read once do
// not push the bias / mask tables (re-read by every unit) out of the L2.
constexpr int kStreamPolicy = 2;

constexpr int kMapMaxN = 1024;   // largest window addressed through a window map: row * win_w must stay below 65536
constexpr int kKeyChunk = 256;   // keys staged in LDS at a time by the query-owning kernels
constexpr int kLdsStride = 40;   // elements per staged row (32 + 8 pad): 80-byte rows

// ---- launch parameters -------------------------------------------------------
struct T4 {
    const void* ptr;
    int64_t sb, sh, sn;
};
// Window partition and cyclic shift as address arithmetic (nw == 0: off, tensors are [BW, H, N, d]).
// With a map, q / k / v / o (and the gradients) are token grids [B, gh * gw, ...]: T4::sb is the stride
// between images, T4::sn the stride between consecutive tokens of the row-major grid, and row n = r ww + c
// of window w = wy nwx + wx of an image sits at grid position ((wy wh + r + sh) mod gh, (wx ww + c + sw) mod gw).
struct WinMap {
    int nw, nwx;        // windows per image, windows per grid row
    int gh, gw;         // token grid of one image
    int wh, ww;         // window extents
    int sh, sw;         // cyclic shift (0 <= sh < gh, 0 <= sw < gw)
    int inv_ww;         // 65536 / ww + 1: n / ww == (n * inv_ww) >> 16 for n * ww < 65536
};
// Element offset of row `row` of unit b, head h.  b is uniform, so the two divisions are scalar work.
template <bool MAPPED>
__device__ __forceinline__ int64_t row_off(const T4& t, const WinMap& m, int b, int h, int row) {
    if (!MAPPED) return b * t.sb + h * t.sh + (int64_t)row * t.sn;
    const int img = b / m.nw, w = b - img * m.nw;
    const int wy = w / m.nwx, wx = w - wy * m.nwx;
    const int r = (row * m.inv_ww) >> 16, c = row - r * m.ww;
    int y = wy * m.wh + r + m.sh;
    int x = wx * m.ww + c + m.sw;
    y -= y >= m.gh ? m.gh : 0;
    x -= x >= m.gw ? m.gw : 0;
    return img * t.sb + h * t.sh + (int64_t)(y * m.gw + x) * t.sn;
}

// The same with the map decided at run time, for the kernels that stream long windows: a few address
// computations per key chunk, so the branch costs nothing there.
__device__ __forceinline__ int64_t row_off_any(const T4& t, const WinMap& m, int b, int h, int row) {
    return m.nw > 0 ? row_off<true>(t, m, b, h, row) : row_off<false>(t, m, b, h, row);
}

// Row `row` of a tensor whose unit starts at `unit` (a wavefront-uniform pointer): one full-rate 24-bit
// multiply and a 32-bit byte offset on the uniform base, instead of the 64-bit multiply-add chain (three
// quarter-rate instructions and two 64-bit adds per address) that `unit + row * sn` costs with 64-bit strides.
// The host checks that rows and row strides stay below 2^24 and their product below 2^31.
template <class E>
__device__ __forceinline__ const E* row_at(const E* unit, int row, int64_t sn, int col = 0) {
    uint32_t prod;      // strides are wavefront-uniform (kernel arguments): src0 may be a scalar register
    asm("v_mul_u32_u24 %0, %1, %2" : "=v"(prod) : "s"((uint32_t)sn), "v"((uint32_t)row));
    const uint32_t boff = (prod + (uint32_t)col) * (uint32_t)sizeof(E);
    return reinterpret_cast<const E*>(reinterpret_cast<const char*>(unit) + boff);
}
// Uniform start of unit b, head h (of its image with a window map) and the row's position inside it.
template <bool MAPPED, class E>
__device__ __forceinline__ const E* unit_ptr(const T4& t, const WinMap& m, int b, int h) {
    const int64_t u = MAPPED ? (int64_t)(b / m.nw) * t.sb : (int64_t)b * t.sb;
    return reinterpret_cast<const E*>(t.ptr) + u + h * t.sh;
}
template <bool MAPPED>
__device__ __forceinline__ int unit_row(const WinMap& m, int b, int row) {
    if (!MAPPED) return row;
    const int w = b % m.nw;
    const int wy = w / m.nwx, wx = w - wy * m.nwx;
    const int r = (row * m.inv_ww) >> 16, c = row - r * m.ww;
    int y = wy * m.wh + r + m.sh;
    int x = wx * m.ww + c + m.sw;
    y -= y >= m.gh ? m.gh : 0;
    x -= x >= m.gw ? m.gw : 0;
    return y * m.gw + x;
}
// The two together: address of row `row` of unit b, head h.
template <bool MAPPED, class E>
__device__ __forceinline__ const E* row_ptr(const T4& t, const WinMap& m, int b, int h, int row, int col = 0) {
    return row_at(unit_ptr<MAPPED, E>(t, m, b, h), unit_row<MAPPED>(m, b, row), t.sn, col);
}

// The two halves of that for a loop over rows: the unit's start (uniform, taken once) and the row's position
// inside it.
__device__ __forceinline__ int64_t unit_off_any(const T4& t, const WinMap& m, int b, int h) {
    return (m.nw > 0 ? (int64_t)(b / m.nw) * t.sb : (int64_t)b * t.sb) + h * t.sh;
}
__device__ __forceinline__ int unit_row_any(const WinMap& m, int b, int row) {
    return m.nw > 0 ? unit_row<true>(m, b, row) : row;
}

struct FwdParams {
    T4 q, k, v, o;
    WinMap map;
    const void* logit_scale;
    const void* bias;
    int64_t bias_sh, bias_sn;
    const void* mask;
    int64_t mask_sw, mask_sn;
    const uint8_t* mask_live;  // [n_windows] flags from the mask scan (0 = window's mask is all zero, bit 0 =
                               // it has a non-zero entry, bit 1 = all entries <= 0 and every row keeps a 0,
                               // bit 2 = the window has a RegionRecord);
                               // nullptr = assume every window live and nothing known about it
    const uint8_t* regions;    // [n_windows] RegionRecord, or nullptr
    float* lse;
    int64_t lse_sb, lse_sh;
    int bw, heads, n, n_windows;
    int scale_kind;
    float default_scale;  // 1/sqrt(head_dim), used when no logit scale is given
    bool side_vec;    // rows of bias and mask may be read with 16-byte loads and n % 8 == 0
    bool side_vec_rows;   // ... or n % 8 != 0 but every row is at least n rounded up to 8 entries long (resident kernels)
    int waves;        // wavefronts per workgroup
    int q_chunks;     // workgroups per (bw, head)
    int cus;          // compute units of the device
    int groups;       // persistent workgroups per head (resident-bias kernel)
};

struct BwdParams {
    T4 q, k, v, o, d_o, dq, dk, dv;
    WinMap map;
    const void* logit_scale;
    const void* bias;
    int64_t bias_sh, bias_sn;
    const void* mask;
    int64_t mask_sw, mask_sn;
    const uint8_t* mask_live;
    const uint8_t* regions;    // [n_windows] RegionRecord, or nullptr
    const float* lse;
    int64_t lse_sb, lse_sh;
    int bw, heads, n, n_windows;
    int scale_kind;
    float default_scale;
    void* dbias;      // [H, N, N] in the input dtype
    void* dscale;     // [H] in the input dtype
    void* workspace;
    int cus;          // compute units of the device
    hipEvent_t ev_start, ev_stop;  // optional: recorded right around the main backward kernel
    // filled in by the launcher
    int waves;        // wavefronts per workgroup = key tiles of 16
    int groups;       // workgroups per head (each walks bw = g, g + groups, ...)
    float* part_dbias;   // [H, db_parts, NP, NQ] fp32, key-major
    int db_parts;        // partial tiles per head: groups per launch of the key-side kernel
    int db_slot0;        // first partial slot of the current launch
    float* part_dscale;  // [H, ds_parts] fp32, one per workgroup of the dq kernel
    int ds_parts;        // partials per head that the reduction sums
    int ds_slot0;        // first partial slot of the current launch of the resident dq kernel
    int dq_groups;       // workgroups per head of the current launch of the resident dq kernel
    float* delta;        // [BW * H, delta_stride] fp32 rowsum(o * dO), written by the key-side kernel
    int delta_stride;
    // windows of more than 256 tokens: 256 x 256 super-tiles of the score matrix
    int n_chunks;        // chunks of 256 rows per side
    int r_tot, npk_tot;  // padded query / key extents of the key-major side tables and partial tiles
    float* part_dk;      // [n_chunks, BW, H, npk_tot, 32] fp32 partials over the query chunks
    float* part_dv;
    int dq_waves;        // wavefronts per workgroup of the dq kernel
    int dq_chunks;       // dq workgroups per (bw, head)
    int big_xcd;         // super-tiled key-side kernel: workgroup order that keeps a (head, group) pair on one XCD
    int dkv_blocks;      // dq launch for windows beyond 256 tokens: groups of 8 workgroups that sum dk / dv partials
    bool side_vec;       // rows of bias and mask (query-major) may be read with 16-byte loads, n % 8 == 0
    bool side_vec_rows;  // ... or n % 8 != 0 but every row is at least n rounded up to 8 entries long (resident kernels)
    const void* bias_t;  // [H, NP, NQ] input dtype: bias transposed to key-major, zero padded
    const void* mask_t;  // [nW, NP, NQ] mask dtype: mask transposed to key-major, zero padded
    const float* tab;    // score tables of the one-pass kernel: (bias + mask) * log2e in accumulator order, slot h for
                         // head h alone and slot heads + w * heads + h for window w with a live mask
};

// dk, dv = sum over the query chunks of the fp32 partials (windows of more than 256 tokens), cast to the input
// dtype.  Four threads per (b, h, key) row, 8 columns each; `block` counts workgroups of `threads` threads.
template <int DT>
__device__ __forceinline__ void dkv_reduce_rows(const BwdParams& p, int64_t block, int threads, int tid) {
    typedef typename Elem<DT>::E E;
    typedef typename Elem<DT>::V8 V8;
    const int64_t rows = (int64_t)p.bw * p.heads * p.n;
    const int64_t i = block * (threads >> 2) + (tid >> 2);
    if (i >= rows) return;
    const int key = (int)(i % p.n);
    const int64_t bh = i / p.n;
    const int h = (int)(bh % p.heads);
    const int64_t b = bh / p.heads;
    const int c8 = (tid & 3) * 8;
    float sk[8], sv[8];
#pragma unroll
    for (int j = 0; j < 8; j++) { sk[j] = 0.f; sv[j] = 0.f; }
    for (int qs = 0; qs < p.n_chunks; qs++) {
        const int64_t row = (((int64_t)qs * p.bw + b) * p.heads + h) * p.npk_tot + key;
#pragma unroll
        for (int v = 0; v < 2; v++) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(p.part_dk + row * 32 + c8 + 4 * v);
            const f32x4 c = *reinterpret_cast<const f32x4*>(p.part_dv + row * 32 + c8 + 4 * v);
#pragma unroll
            for (int j = 0; j < 4; j++) { sk[4 * v + j] += a[j]; sv[4 * v + j] += c[j]; }
        }
    }
    V8 ok, ov;
#pragma unroll
    for (int j = 0; j < 8; j++) { ok[j] = (E)sk[j]; ov[j] = (E)sv[j]; }
    st8<V8>(reinterpret_cast<E*>(const_cast<void*>(p.dk.ptr)) + row_off_any(p.dk, p.map, (int)b, h, key) + c8, ok);
    st8<V8>(reinterpret_cast<E*>(const_cast<void*>(p.dv.ptr)) + row_off_any(p.dv, p.map, (int)b, h, key) + c8, ov);
}

}  // namespace fwa2
