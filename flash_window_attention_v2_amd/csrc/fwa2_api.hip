// extern "C" surface of libfwa2 (declared in include/fwa2.h): argument
// validation, workspace sizing and dispatch to the gfx950 kernels.  Nothing
// here allocates device memory or synchronises.
#include <atomic>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fwa2_common.hpp"

namespace fwa2 {
hipError_t launch_forward(FwdParams p, int dtype, bool has_bias, int mask_dt, hipStream_t st);
hipError_t launch_mask_scan(const void* mask, int mask_dt, int64_t sw, int64_t sn, int n, int n_windows,
                            uint8_t* live, uint8_t* regions, hipStream_t st);
static_assert(sizeof(RegionRecord) == FWA2_MASK_REGION_BYTES, "the header states the size of a region record");
hipError_t launch_backward(const BwdParams& p, int dtype, bool has_bias, int mask_dt, hipStream_t st);
size_t backward_workspace_bytes(int heads, int n, int bw, bool has_bias, bool has_mask, int n_windows, int cus);
bool generic_problem(int d, int n, int nk);
size_t generic_workspace_bytes(int heads, int n, int nk, int bw, bool has_bias);
hipError_t launch_generic(const fwa2_problem* p, bool backward);
int backward_supported(int n);
hipError_t launch_cpb_bias_forward(const void* table, int dtype, int heads, int wh, int ww, void* bias, hipStream_t st);
hipError_t launch_cpb_bias_backward(const void* table, const void* dbias, int dtype, int heads, int wh, int ww,
                                    void* dtable, hipStream_t st);
}  // namespace fwa2

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_t4(const char* name, const fwa2_tensor4& t, int head_dim) {
    if (t.ptr == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: null pointer", name);
    if (!aligned16(t.ptr) || (t.stride_bw % 8) || (t.stride_h % 8) || (t.stride_n % 8))
        return fail(FWA2_ERR_UNSUPPORTED,
                    "%s: rows must start on 16-byte boundaries (pointer 16-byte aligned, strides multiples of 8 elements)",
                    name);
    if (t.stride_n >= (1 << 24))
        return fail(FWA2_ERR_UNSUPPORTED, "%s: row stride %lld is beyond the 2^24 elements the kernels address rows with", name,
                    (long long)t.stride_n);
    if (t.stride_n < head_dim) return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: row stride %lld overlaps rows", name, (long long)t.stride_n);
    return FWA2_OK;
}

fwa2::T4 to_t4(const fwa2_tensor4& t) { return fwa2::T4{t.ptr, t.stride_bw, t.stride_h, t.stride_n}; }

// Compute units of the CURRENT device, asked once per device (a property query: no device memory is touched and
// nothing is launched).  Without a visible device the MI355X's 256 are assumed, so that a host-only caller of
// fwa2_validate / fwa2_backward_workspace_bytes sees the sizes of the part this library is written for.
constexpr int kMaxDevices = 64;
std::atomic<int> g_cus[kMaxDevices];
int cu_count() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    n = g_cus[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    g_cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

// ---- scratch of the allocation-free backward entry point ----
// One copy of this array exists on every GPU the library is loaded on and stays there until the process ends.
// Host code never uses the array's name as an address: scratch_of_current_device() asks the runtime for the
// address of the current device's copy, once per device, and every later use goes through that pointer.
constexpr size_t kStaticScratchBytes = FWA2_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices];

int scratch_of_current_device(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return fail(FWA2_ERR_NO_DEVICE, "fwa2_backward_static: no current device");
    if (dev < 0 || dev >= kMaxDevices)
        return fail(FWA2_ERR_UNSUPPORTED, "fwa2_backward_static: device index %d is beyond the %d this library tracks", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(FWA2_ERR_HIP, "fwa2_backward_static: address of the scratch array on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return FWA2_OK;
}

int validate(const fwa2_problem* p, int backward) {
    if (p == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "problem is null");
    if (p->struct_bytes != sizeof(fwa2_problem) || p->abi_version != FWA2_ABI_VERSION)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "fwa2_problem layout mismatch: caller %u bytes / abi %u, library %zu bytes / abi %d",
                    p->struct_bytes, p->abi_version, sizeof(fwa2_problem), FWA2_ABI_VERSION);
    if (p->dtype != FWA2_F16 && p->dtype != FWA2_BF16)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "Only support fp16 and bf16");
    if (p->bw <= 0 || p->heads <= 0 || p->n <= 0 || p->head_dim <= 0)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "bw, heads, n and head_dim must be positive");
    if (p->head_dim > 128)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "FlashAttention only support head dimensions up to 128");
    if (p->head_dim % 8)
        return fail(FWA2_ERR_UNSUPPORTED, "head_dim %d: head dimensions must be multiples of 8 (16-byte row chunks)", p->head_dim);
    if ((int64_t)p->bw * p->heads * ((p->n + 255) / 256) > 0x7fffffffLL)
        return fail(FWA2_ERR_UNSUPPORTED, "too many (batch*window, head) pairs for one launch");
    int rc;
    const int hd = p->head_dim;
    if ((rc = check_t4("q", p->q, hd)) || (rc = check_t4("k", p->k, hd)) || (rc = check_t4("v", p->v, hd)) || (rc = check_t4("o", p->o, hd)))
        return rc;
    if (p->scale_kind == FWA2_SCALE_TENSOR) {
        if (p->logit_scale == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "logit_scale: null with FWA2_SCALE_TENSOR");
    } else if (p->scale_kind != FWA2_SCALE_DEFAULT) {
        return fail(FWA2_ERR_INVALID_ARGUMENT, "scale_kind %d unknown", p->scale_kind);
    }
    {
        // rows inside a unit (an image with a window map) are addressed with 32-bit byte offsets
        const int64_t rows = p->grid_h > 0 ? (int64_t)p->grid_h * p->grid_w : (p->n_keys > p->n ? p->n_keys : p->n);
        const fwa2_tensor4* ts[] = {&p->q, &p->k, &p->v, &p->o, &p->d_o, &p->dq, &p->dk, &p->dv};
        for (int i = 0; i < (backward ? 8 : 4); i++)
            if (rows >= (1 << 24) || rows * ts[i]->stride_n >= (1LL << 30))
                return fail(FWA2_ERR_UNSUPPORTED, "a unit spans more than 2^31 bytes (rows %lld, row stride %lld)", (long long)rows,
                            (long long)ts[i]->stride_n);
    }
    if (p->n_keys < 0) return fail(FWA2_ERR_INVALID_ARGUMENT, "n_keys must not be negative");
    if (p->scale_head_dim < 0 || p->scale_head_dim > p->head_dim)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "scale_head_dim must be 0 or a dimension up to head_dim (rows padded with zeros)");
    const int nk = p->n_keys > 0 ? p->n_keys : p->n;
    if (p->bias.ptr && p->bias.stride_n < nk)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "bias: row stride %lld < number of keys", (long long)p->bias.stride_n);
    if (p->mask.ptr) {
        if (p->mask_dtype != p->dtype && p->mask_dtype != FWA2_F32)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "mask dtype must be the input dtype or fp32");
        if (p->n_windows <= 0 || p->bw % p->n_windows)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "bw %d is not a multiple of n_windows %d", p->bw, p->n_windows);
        if (p->mask.stride_n < nk)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "mask: row stride %lld < number of keys", (long long)p->mask.stride_n);
    }
    if (p->grid_h != 0 || p->grid_w != 0 || p->win_h != 0 || p->win_w != 0 || p->shift_h != 0 || p->shift_w != 0) {
        if (p->grid_h <= 0 || p->grid_w <= 0 || p->win_h <= 0 || p->win_w <= 0 || p->grid_h % p->win_h || p->grid_w % p->win_w)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "window map: the %d x %d grid is not a whole number of %d x %d windows",
                        p->grid_h, p->grid_w, p->win_h, p->win_w);
        if (p->n != p->win_h * p->win_w)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "window map: n = %d is not win_h * win_w", p->n);
        if (p->shift_h < 0 || p->shift_h >= p->grid_h || p->shift_w < 0 || p->shift_w >= p->grid_w)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "window map: shifts must lie in [0, grid extent)");
        const int nw = (p->grid_h / p->win_h) * (p->grid_w / p->win_w);
        if (p->bw % nw) return fail(FWA2_ERR_INVALID_ARGUMENT, "window map: bw %d is not a multiple of %d windows per image", p->bw, nw);
        if (p->mask.ptr && p->n_windows != nw)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "window map: mask has %d windows, the grid %d", p->n_windows, nw);
        if (nk != p->n)
            return fail(FWA2_ERR_UNSUPPORTED, "window map: needs as many keys as queries");
        if (p->win_w > 64 || p->n > fwa2::kMapMaxN)
            return fail(FWA2_ERR_UNSUPPORTED, "window map: windows of more than %d tokens (or wider than 64) are not supported",
                        fwa2::kMapMaxN);
    }
    if ((p->ev_start == nullptr) != (p->ev_stop == nullptr))
        return fail(FWA2_ERR_INVALID_ARGUMENT, "ev_start and ev_stop: give both events or neither");
    if (p->lse == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "lse: null pointer");
    if (p->lse_stride_h < p->n) return fail(FWA2_ERR_INVALID_ARGUMENT, "lse: head stride %lld < n", (long long)p->lse_stride_h);
    if (backward) {
        if ((rc = check_t4("do", p->d_o, hd)) || (rc = check_t4("dq", p->dq, hd)) || (rc = check_t4("dk", p->dk, hd)) ||
            (rc = check_t4("dv", p->dv, hd)))
            return rc;
        if (p->bias.ptr && p->dbias == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "dbias: null although bias is given");
        if (p->scale_kind == FWA2_SCALE_TENSOR && p->dscale == nullptr)
            return fail(FWA2_ERR_INVALID_ARGUMENT, "dscale: null although logit_scale is given");
        if (!fwa2::backward_supported(p->n))
            return fail(FWA2_ERR_UNSUPPORTED, "backward: n = %d is not supported by this build", p->n);
        const size_t need = fwa2_backward_workspace_bytes(p);
        if (need && (p->workspace == nullptr || p->workspace_bytes < need))
            return fail(FWA2_ERR_INVALID_ARGUMENT, "workspace: need %zu bytes, got %zu", need, p->workspace_bytes);
        if (need && (reinterpret_cast<uintptr_t>(p->workspace) & 255))
            return fail(FWA2_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
    }
    return FWA2_OK;
}

fwa2::WinMap to_map(const fwa2_problem* p) {
    fwa2::WinMap m;
    memset(&m, 0, sizeof(m));
    if (p->grid_h > 0) {
        m.nwx = p->grid_w / p->win_w;
        m.nw = (p->grid_h / p->win_h) * m.nwx;
        m.gh = p->grid_h; m.gw = p->grid_w;
        m.wh = p->win_h; m.ww = p->win_w;
        m.sh = p->shift_h; m.sw = p->shift_w;
        m.inv_ww = 65536 / p->win_w + 1;
    }
    return m;
}

bool row_vec_ok(const void* ptr, int64_t sa, int64_t sn, int n) {
    return aligned16(ptr) && (sa % 8) == 0 && (sn % 8) == 0 && (n % 8) == 0;
}
// Rows that start on 16-byte boundaries and are long enough for whole groups of 8 entries, whatever n is (the
// caller padded them): the entries beyond n are never used.
bool row_groups_ok(const void* ptr, int64_t sa, int64_t sn, int n) {
    return aligned16(ptr) && (sa % 8) == 0 && (sn % 8) == 0 && sn >= ((n + 7) & ~7);
}

}  // namespace

extern "C" {

int fwa2_abi_version(void) { return FWA2_ABI_VERSION; }

const char* fwa2_last_error(void) { return g_err; }

int fwa2_validate(const fwa2_problem* p, int backward) {
    g_err[0] = 0;
    return validate(p, backward);
}

size_t fwa2_backward_workspace_bytes(const fwa2_problem* p) {
    if (p == nullptr) return 0;
    // sizes fwa2_validate refuses: nothing to reserve
    if (p->bw <= 0 || p->heads <= 0 || p->n <= 0 || p->head_dim <= 0 || p->n_keys < 0) return 0;
    if (p->mask.ptr != nullptr && (p->n_windows <= 0 || p->n_windows > p->bw)) return 0;
    {
        // sizes no device can hold (the partial tiles of dbias, the partial sums of dk / dv): answered without
        // forming the products, which would wrap
        const double n = p->n, nk = p->n_keys > 0 ? p->n_keys : p->n, units = (double)p->bw * p->heads;
        if (p->heads * n * (n > nk ? n : nk) > 0x1p44 || units * n * (n > nk ? n : nk) > 0x1p52) return SIZE_MAX;
    }
    if (fwa2::generic_problem(p->head_dim, p->n, p->n_keys > 0 ? p->n_keys : p->n))
        return fwa2::generic_workspace_bytes(p->heads, p->n, p->n_keys > 0 ? p->n_keys : p->n, p->bw, p->bias.ptr != nullptr);
    return fwa2::backward_workspace_bytes(p->heads, p->n, p->bw, p->bias.ptr != nullptr, p->mask.ptr != nullptr,
                                          p->n_windows, cu_count());
}

static int mask_scan(const char* what, const void* mask, int mask_dtype, int n_windows, int n, int64_t stride_w,
                     int64_t stride_n, uint8_t* live, void* regions, bool want_regions, void* stream) {
    g_err[0] = 0;
    if (mask == nullptr || live == nullptr || n_windows <= 0 || n <= 0 || (want_regions && regions == nullptr))
        return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: bad argument", what);
    if (want_regions && ((uintptr_t)regions & 15))
        return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: regions must be 16-byte aligned", what);
    if (mask_dtype != FWA2_F16 && mask_dtype != FWA2_BF16 && mask_dtype != FWA2_F32)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: bad mask dtype", what);
    hipError_t e = fwa2::launch_mask_scan(mask, mask_dtype, stride_w, stride_n, n, n_windows, live, (uint8_t*)regions,
                                          (hipStream_t)stream);
    if (e != hipSuccess) return fail(FWA2_ERR_HIP, "mask scan launch: %s", hipGetErrorString(e));
    return FWA2_OK;
}

int fwa2_mask_scan(const void* mask, int mask_dtype, int n_windows, int n, int64_t stride_w, int64_t stride_n,
                   uint8_t* live, void* stream) {
    return mask_scan("fwa2_mask_scan", mask, mask_dtype, n_windows, n, stride_w, stride_n, live, nullptr, false, stream);
}

int fwa2_mask_scan_regions(const void* mask, int mask_dtype, int n_windows, int n, int64_t stride_w, int64_t stride_n,
                           uint8_t* live, void* regions, void* stream) {
    return mask_scan("fwa2_mask_scan_regions", mask, mask_dtype, n_windows, n, stride_w, stride_n, live, regions, true,
                     stream);
}

static int check_cpb(const char* what, const void* a, const void* b, const void* c, int dtype, int heads, int wh, int ww) {
    if (a == nullptr || b == nullptr || c == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
    if (dtype != FWA2_F16 && dtype != FWA2_BF16) return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: dtype must be fp16 or bf16", what);
    if (heads <= 0 || wh <= 0 || ww <= 0) return fail(FWA2_ERR_INVALID_ARGUMENT, "%s: heads and window extents must be positive", what);
    if ((int64_t)wh * ww > 46340) return fail(FWA2_ERR_UNSUPPORTED, "%s: window of %d x %d tokens is too large", what, wh, ww);
    return FWA2_OK;
}

int fwa2_cpb_bias_forward(const void* table, int dtype, int heads, int wh, int ww, void* bias, void* stream) {
    g_err[0] = 0;
    int rc = check_cpb("fwa2_cpb_bias_forward", table, bias, bias, dtype, heads, wh, ww);
    if (rc) return rc;
    hipError_t e = fwa2::launch_cpb_bias_forward(table, dtype, heads, wh, ww, bias, (hipStream_t)stream);
    if (e != hipSuccess) return fail(FWA2_ERR_HIP, "cpb bias forward launch: %s", hipGetErrorString(e));
    return FWA2_OK;
}

int fwa2_cpb_bias_backward(const void* table, const void* dbias, int dtype, int heads, int wh, int ww, void* dtable,
                           void* stream) {
    g_err[0] = 0;
    int rc = check_cpb("fwa2_cpb_bias_backward", table, dbias, dtable, dtype, heads, wh, ww);
    if (rc) return rc;
    hipError_t e = fwa2::launch_cpb_bias_backward(table, dbias, dtype, heads, wh, ww, dtable, (hipStream_t)stream);
    if (e != hipSuccess) return fail(FWA2_ERR_HIP, "cpb bias backward launch: %s", hipGetErrorString(e));
    return FWA2_OK;
}

int fwa2_forward(const fwa2_problem* p) {
    g_err[0] = 0;
    int rc = validate(p, 0);
    if (rc) return rc;
    const bool timed = p->ev_start != nullptr && p->ev_stop != nullptr;
    if (fwa2::generic_problem(p->head_dim, p->n, p->n_keys > 0 ? p->n_keys : p->n)) {
        if (timed) (void)hipEventRecord((hipEvent_t)p->ev_start, (hipStream_t)p->stream);
        hipError_t eg = fwa2::launch_generic(p, false);
        if (timed) (void)hipEventRecord((hipEvent_t)p->ev_stop, (hipStream_t)p->stream);
        if (eg != hipSuccess) return fail(FWA2_ERR_HIP, "forward launch: %s", hipGetErrorString(eg));
        return FWA2_OK;
    }
    fwa2::FwdParams k;
    memset(&k, 0, sizeof(k));
    k.q = to_t4(p->q); k.k = to_t4(p->k); k.v = to_t4(p->v); k.o = to_t4(p->o);
    k.map = to_map(p);
    k.logit_scale = p->logit_scale;
    k.bias = p->bias.ptr; k.bias_sh = p->bias.stride_a; k.bias_sn = p->bias.stride_n;
    k.mask = p->mask.ptr; k.mask_sw = p->mask.stride_a; k.mask_sn = p->mask.stride_n;
    // the kernels keep the per-window flags in LDS; beyond that many windows they go without
    k.mask_live = (p->mask.ptr && p->n_windows <= fwa2::kLiveCache) ? p->mask_live : nullptr;
    k.regions = k.mask_live ? (const uint8_t*)p->mask_regions : nullptr;
    k.lse = p->lse; k.lse_sb = p->lse_stride_bw; k.lse_sh = p->lse_stride_h;
    k.bw = p->bw; k.heads = p->heads; k.n = p->n; k.n_windows = p->mask.ptr ? p->n_windows : 1;
    k.scale_kind = p->scale_kind;
    k.default_scale = 1.0f / sqrtf((float)(p->scale_head_dim > 0 ? p->scale_head_dim : p->head_dim));
    k.side_vec = (!p->bias.ptr || row_vec_ok(p->bias.ptr, p->bias.stride_a, p->bias.stride_n, p->n)) &&
                 (!p->mask.ptr || row_vec_ok(p->mask.ptr, p->mask.stride_a, p->mask.stride_n, p->n));
    k.side_vec_rows = (!p->bias.ptr || row_groups_ok(p->bias.ptr, p->bias.stride_a, p->bias.stride_n, p->n)) &&
                      (!p->mask.ptr || row_groups_ok(p->mask.ptr, p->mask.stride_a, p->mask.stride_n, p->n));
    k.cus = cu_count();
    if (timed) (void)hipEventRecord((hipEvent_t)p->ev_start, (hipStream_t)p->stream);
    hipError_t e = fwa2::launch_forward(k, p->dtype, p->bias.ptr != nullptr, p->mask.ptr ? p->mask_dtype : -1,
                                        (hipStream_t)p->stream);
    if (timed) (void)hipEventRecord((hipEvent_t)p->ev_stop, (hipStream_t)p->stream);
    if (e != hipSuccess) return fail(FWA2_ERR_HIP, "forward launch: %s", hipGetErrorString(e));
    return FWA2_OK;
}

static int run_backward(const fwa2_problem* p) {
    int rc = validate(p, 1);
    if (rc) return rc;
    if (fwa2::generic_problem(p->head_dim, p->n, p->n_keys > 0 ? p->n_keys : p->n)) {
        hipError_t eg = fwa2::launch_generic(p, true);
        if (eg != hipSuccess) return fail(FWA2_ERR_HIP, "backward launch: %s", hipGetErrorString(eg));
        return FWA2_OK;
    }
    fwa2::BwdParams k;
    memset(&k, 0, sizeof(k));
    k.q = to_t4(p->q); k.k = to_t4(p->k); k.v = to_t4(p->v); k.o = to_t4(p->o);
    k.d_o = to_t4(p->d_o); k.dq = to_t4(p->dq); k.dk = to_t4(p->dk); k.dv = to_t4(p->dv);
    k.map = to_map(p);
    k.logit_scale = p->logit_scale;
    k.bias = p->bias.ptr; k.bias_sh = p->bias.stride_a; k.bias_sn = p->bias.stride_n;
    k.mask = p->mask.ptr; k.mask_sw = p->mask.stride_a; k.mask_sn = p->mask.stride_n;
    // the kernels keep the per-window flags in LDS; beyond that many windows they go without
    k.mask_live = (p->mask.ptr && p->n_windows <= fwa2::kLiveCache) ? p->mask_live : nullptr;
    k.regions = k.mask_live ? (const uint8_t*)p->mask_regions : nullptr;
    k.lse = p->lse; k.lse_sb = p->lse_stride_bw; k.lse_sh = p->lse_stride_h;
    k.bw = p->bw; k.heads = p->heads; k.n = p->n; k.n_windows = p->mask.ptr ? p->n_windows : 1;
    k.scale_kind = p->scale_kind;
    k.default_scale = 1.0f / sqrtf((float)(p->scale_head_dim > 0 ? p->scale_head_dim : p->head_dim));
    k.dbias = p->dbias; k.dscale = p->dscale;
    k.side_vec = (!p->bias.ptr || row_vec_ok(p->bias.ptr, p->bias.stride_a, p->bias.stride_n, p->n)) &&
                 (!p->mask.ptr || row_vec_ok(p->mask.ptr, p->mask.stride_a, p->mask.stride_n, p->n));
    k.side_vec_rows = (!p->bias.ptr || row_groups_ok(p->bias.ptr, p->bias.stride_a, p->bias.stride_n, p->n)) &&
                      (!p->mask.ptr || row_groups_ok(p->mask.ptr, p->mask.stride_a, p->mask.stride_n, p->n));
    k.workspace = p->workspace;
    k.cus = cu_count();
    if (p->ev_start != nullptr && p->ev_stop != nullptr) {
        k.ev_start = (hipEvent_t)p->ev_start;
        k.ev_stop = (hipEvent_t)p->ev_stop;
    }
    hipError_t e = fwa2::launch_backward(k, p->dtype, p->bias.ptr != nullptr, p->mask.ptr ? p->mask_dtype : -1,
                                         (hipStream_t)p->stream);
    if (e != hipSuccess) return fail(FWA2_ERR_HIP, "backward launch: %s", hipGetErrorString(e));
    return FWA2_OK;
}

int fwa2_backward(const fwa2_problem* p) {
    g_err[0] = 0;
    return run_backward(p);
}

int fwa2_backward_static(const fwa2_problem* p) {
    g_err[0] = 0;
    if (p == nullptr) return fail(FWA2_ERR_INVALID_ARGUMENT, "problem is null");
    if (p->struct_bytes != sizeof(fwa2_problem) || p->abi_version != FWA2_ABI_VERSION)
        return fail(FWA2_ERR_INVALID_ARGUMENT, "fwa2_problem layout mismatch: caller %u bytes / abi %u, library %zu bytes / abi %d",
                    p->struct_bytes, p->abi_version, sizeof(fwa2_problem), FWA2_ABI_VERSION);
    int rc = validate(p, 0);      // sizes and dtypes are sane before the workspace is sized from them
    if (rc) return rc;
    const size_t need = fwa2_backward_workspace_bytes(p);
    if (need > kStaticScratchBytes)
        return fail(FWA2_ERR_UNSUPPORTED,
                    "fwa2_backward_static: this problem needs %zu bytes of scratch, the library's static buffer holds %zu; "
                    "use fwa2_backward with a caller-owned workspace", need, kStaticScratchBytes);
    void* ptr = nullptr;
    rc = scratch_of_current_device(&ptr);
    if (rc) return rc;
    fwa2_problem q = *p;
    q.workspace = ptr;
    q.workspace_bytes = kStaticScratchBytes;
    return run_backward(&q);
}

}  // extern "C"
