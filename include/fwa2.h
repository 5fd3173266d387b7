/*
 * fwa2.h -- C ABI of libfwa2: Swin V2 scaled-cosine window attention,
 * forward and backward, as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The library replaces the two host launchers of the reference
 * implementation and the Triton kernels behind them:
 *
 *   fwa2_forward   <->  _flash_attn_forward
 *                       flash_win_attn_v2/kernels/attn_kernel_forward.py:261-345
 *                       (kernel _fwd_kernel, :33-258)
 *   fwa2_backward  <->  _flash_attn_backward
 *                       flash_win_attn_v2/kernels/attn_kernel_backward.py:567-711
 *                       (kernels _bwd_preprocess_do_o_dot :6-51, _bwd_kernel :389-564)
 *
 * Conventions
 *   - plain pointers and sizes only; no framework types cross this boundary.
 *   - the library allocates nothing and keeps no pointer after a call returns;
 *     every buffer, including workspaces, belongs to the caller.
 *   - every call only enqueues work on `stream` (a hipStream_t, NULL = the
 *     default stream) and never synchronises the device.
 *   - strides are in ELEMENTS of the tensor's own type; the innermost (head
 *     dim) stride of q, k, v, o, do, dq, dk, dv is 1 and is not passed.  The
 *     other three strides are free, as in the reference
 *     (flash_window_attention_v2.py:20, attn_kernel_forward.py:313-328),
 *     within these bounds: row strides multiples of 8 elements and below
 *     2^24, and one unit (a window's rows, or a whole image's token grid with
 *     a window map) spanning less than 2^31 bytes, since rows inside a unit
 *     are addressed with 32-bit offsets; unit and head strides are 64-bit.
 *   - all functions are re-entrant; the error string is thread-local.
 *   - return value 0 = FWA2_OK, otherwise an fwa2_status; fwa2_last_error()
 *     then describes the failure.
 */
#ifndef FWA2_H
#define FWA2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FWA2_ABI_VERSION 4

typedef enum fwa2_status {
    FWA2_OK = 0,
    FWA2_ERR_INVALID_ARGUMENT = 1, /* contract violation (the reference's AssertionError) */
    FWA2_ERR_UNSUPPORTED = 2,      /* legal for the reference, not built here (e.g. head dim % 8 != 0) */
    FWA2_ERR_HIP = 3,              /* a HIP runtime call failed */
    FWA2_ERR_NO_DEVICE = 4         /* no gfx950 device available for the launch */
} fwa2_status;

typedef enum fwa2_dtype {
    FWA2_F16 = 0,
    FWA2_BF16 = 1,
    FWA2_F32 = 2 /* only valid as mask_dtype (attn_kernel_forward.py:287) */
} fwa2_dtype;

typedef enum fwa2_scale_kind {
    FWA2_SCALE_DEFAULT = 0, /* no logit scale given: scores * 1/sqrt(d)  (flash_window_attention_v2.py:14-17) */
    FWA2_SCALE_TENSOR = 1   /* logit_scale[H] given: scores * exp(min(l_h, ln 100)) (attn_kernel_forward.py:118-121) */
} fwa2_scale_kind;

/* A [BW, H, N, d] tensor with unit innermost stride. */
typedef struct fwa2_tensor4 {
    void*   ptr;
    int64_t stride_bw;
    int64_t stride_h;
    int64_t stride_n;
} fwa2_tensor4;

/* A [A, N, N] tensor (bias: A = H, mask: A = nW) with unit innermost stride.  stride_n >= N; the elements of a
 * row past its N-th are never used.  The kernels read bias and mask with 16-byte loads when ptr is 16-byte
 * aligned, both strides are multiples of 8 elements and stride_n >= N rounded up to a multiple of 8; a caller
 * whose N is not a multiple of 8 gets that path by padding the rows (with anything), and the element-wise path
 * otherwise.  On the 16-byte path EVERY row, the last row of the last head or window included, is read up to
 * N rounded up to a multiple of 8: the allocation behind ptr must cover (A - 1) * stride_a + (N - 1) * stride_n
 * + roundup8(N) elements.  A view that ends exactly at its N-th element of the last row must either be padded
 * or be described with a stride_n that is not a multiple of 8 (which selects the element-wise path). */
typedef struct fwa2_tensor3 {
    void*   ptr;       /* NULL = absent */
    int64_t stride_a;
    int64_t stride_n;
} fwa2_tensor3;

/*
 * One operator call.  The same description serves forward and backward; the
 * fields marked (bwd) are ignored by fwa2_forward.
 */
typedef struct fwa2_problem {
    uint32_t struct_bytes;   /* sizeof(fwa2_problem) as the caller compiled it */
    uint32_t abi_version;    /* FWA2_ABI_VERSION */

    int32_t dtype;           /* fwa2_dtype of q,k,v,o,do,dq,dk,dv,bias,logit_scale,dbias,dscale: F16 or BF16 */
    int32_t mask_dtype;      /* fwa2_dtype of mask: == dtype or F32 */
    int32_t scale_kind;      /* fwa2_scale_kind */
    int32_t bw;              /* batch * windows-per-image */
    int32_t heads;
    int32_t n;               /* tokens per window (queries == keys) */
    int32_t head_dim;        /* multiple of 8, at most 128 (see scale_head_dim for others); 32 runs on the tuned kernels */
    int32_t n_windows;       /* leading extent of mask; window of row b is b % n_windows; 1 if no mask */

    fwa2_tensor4 q, k, v;    /* inputs */
    fwa2_tensor4 o;          /* forward: output.  backward: the saved forward output */
    const void*  logit_scale;/* [H] elements of `dtype`, stride 1; NULL unless FWA2_SCALE_TENSOR */
    fwa2_tensor3 bias;       /* [H, N, N] of `dtype`, or ptr NULL */
    fwa2_tensor3 mask;       /* [nW, N, N] of `mask_dtype`, or ptr NULL */
    const uint8_t* mask_live;/* optional [nW] flag bytes from fwa2_mask_scan: 0 = that window's mask is all
                                zero and is skipped; NULL = every window's mask is read */

    float*  lse;             /* [BW, H, lse_stride_h] fp32 natural-log log-sum-exp per query row;
                                written by forward, read by backward (attn_kernel_forward.py:294-295) */
    int64_t lse_stride_bw;
    int64_t lse_stride_h;    /* >= n; the reference rounds N up to a multiple of 64 */

    /* (bwd) */
    fwa2_tensor4 d_o;        /* upstream gradient of o */
    fwa2_tensor4 dq, dk, dv; /* outputs, `dtype` */
    void*   dbias;           /* [H, N, N] contiguous, `dtype`; NULL when bias is absent */
    void*   dscale;          /* [H] contiguous, `dtype`; NULL unless FWA2_SCALE_TENSOR.  Already
                                multiplied by [l_h <= ln 100] (attn_kernel_backward.py:706-711) */
    void*   workspace;       /* device scratch of at least fwa2_backward_workspace_bytes() bytes,
                                256-byte aligned; contents need not be initialised */
    size_t  workspace_bytes;

    void*   stream;          /* hipStream_t */

    /*
     * Optional window map, all zero = off.  It does the cyclic shift and the window partition / reverse of
     * the caller (flash_win_attn_v2/swin_transformer_v2.py:419-441: roll, window_partition, window_reverse,
     * roll back) by address arithmetic.  With grid_h > 0 the tensors q, k, v, o, d_o, dq, dk, dv are token
     * grids [B, grid_h * grid_w, ...] instead of [BW, H, N, d]: stride_bw is then the stride between IMAGES
     * and stride_n the stride between consecutive tokens of the row-major grid.  Unit b = image * nW + window,
     * nW = (grid_h / win_h) (grid_w / win_w), window = wy (grid_w / win_w) + wx; its row n = r win_w + c is the
     * token at ((wy win_h + r + shift_h) mod grid_h, (wx win_w + c + shift_w) mod grid_w).  n must equal
     * win_h win_w and bw must equal B nW; lse, bias, mask, dbias are indexed as without a map (mask: nW == n_windows).
     * Supported for n <= 1024 and win_w <= 64 (FWA2_ERR_UNSUPPORTED otherwise).
     */
    int32_t grid_h, grid_w;
    int32_t win_h, win_w;
    int32_t shift_h, shift_w;

    /*
     * Keys (rows of k and v) per unit when they differ from the n queries, which the reference's kernels allow
     * (attn_kernel_forward.py:263-264) although none of its callers does; 0 = n.  bias is then [H, n, n_keys],
     * mask [nW, n, n_keys], lse and the q-side tensors keep n rows, dk / dv have n_keys rows.  Runs on the plain
     * kernels that also serve head dimensions other than 32; not combined with a window map.
     */
    int32_t n_keys;
    /*
     * Head dimension the default scale 1/sqrt(d) refers to, for rows that were zero-padded up to a multiple of 8
     * (the reference pads to the next power of two inside its kernels and keeps 1/sqrt(d) of the true d,
     * attn_kernel_forward.py:267,298; flash_window_attention_v2.py:14-17); 0 = head_dim.  Zero columns change
     * neither the normalised vectors nor the products, so a caller may pad q, k, v, d_o and slice o, dq, dk, dv.
     */
    int32_t scale_head_dim;

    const void* mask_regions;/* optional [nW] records of FWA2_MASK_REGION_BYTES each from fwa2_mask_scan_regions,
                                given together with the mask_live it filled; NULL = none.  A window flagged there
                                as having region form is then computed from its record (N bytes) instead of its
                                N x N mask entries, by the kernels for windows of up to 256 tokens at head
                                dimension 32; everywhere else the record is ignored and the mask is read */

    /*
     * Optional measurement hook, no counterpart in the reference: two hipEvent_t handles (both or neither) that
     * THIS call records on `stream`.  fwa2_forward records them around its kernels; fwa2_backward and
     * fwa2_backward_static right before and after the main backward kernel (the table / transposing pre-pass and
     * the partial-sum reduction stay outside), so a benchmark can time that kernel alone without a profiler.
     * NULL = nothing is recorded.  The handles belong to the caller; nothing outlives the call.
     */
    void* ev_start;
    void* ev_stop;
} fwa2_problem;

/* Library / ABI identification.  Returns FWA2_ABI_VERSION. */
int fwa2_abi_version(void);

/* Thread-local description of the last failure on the calling thread ("" if none). */
const char* fwa2_last_error(void);

/*
 * Checks a problem description against the contract (shapes, dtypes, strides,
 * NULL-ness, supported sizes) without reading device memory or launching
 * anything.  `backward` non-zero also checks the (bwd) fields, among them the
 * workspace size, which depends on the compute-unit count of the CURRENT
 * device: that one property is asked from the runtime (once per device); a
 * process without a visible device gets the sizes of a 256-CU part (MI355X).
 * Mirrors the assertions at attn_kernel_forward.py:263-292 and
 * attn_kernel_backward.py:571-579, 616-633.
 */
int fwa2_validate(const fwa2_problem* p, int backward);

/*
 * One byte of flags per window (device memory): live[w] = 0 if mask[w] is all
 * zero; otherwise bit 0 is set, and bit 1 is set too when no entry is positive
 * and every row keeps at least one exact zero (the mask only removes keys and
 * never a whole row, as shifted-window masks do).  Shifted-window masks are all
 * zero for most windows; passing the result as fwa2_problem.mask_live lets the
 * kernels skip those reads and pick a cheaper softmax for the rest.
 * Has no counterpart in the reference, which always reads the mask.
 */
int fwa2_mask_scan(const void* mask, int mask_dtype, int n_windows, int n, int64_t stride_w, int64_t stride_n,
                   uint8_t* live, void* stream);

/*
 * fwa2_mask_scan that also recognises the form the reference's mask builder produces
 * (flash_win_attn_v2/swin_transformer_v2.py:386-405: region ids painted on the shifted grid, then
 * mask[w][i][j] = -100 where id_i != id_j, 0 elsewhere).  For a window of n <= 256 tokens whose mask is EXACTLY
 * c * [id_i != id_j] for one finite c < 0 and at most 8 distinct ids (every entry is compared), bit 2 of live[w]
 * is set as well and regions[w] receives c and the n ids; such a window is then attended from those n bytes
 * (see fwa2_problem.mask_regions).  Any other mask keeps bit 2 clear and is read entry by entry as before, so the
 * result is the same for every mask.  `regions` is device memory of n_windows * FWA2_MASK_REGION_BYTES bytes,
 * 16-byte aligned; its layout is private to the library.  Has no counterpart in the reference.
 */
#define FWA2_MASK_REGION_BYTES 272
int fwa2_mask_scan_regions(const void* mask, int mask_dtype, int n_windows, int n, int64_t stride_w, int64_t stride_n,
                           uint8_t* live, void* regions, void* stream);

/*
 * Bytes of device scratch fwa2_backward needs for this problem on the CURRENT
 * device (fp32 accumulators for dbias and dscale; the reference allocates these
 * as db_accum / dscale_accum, attn_kernel_backward.py:609-626).  0 if none, or
 * if bw, heads, n, head_dim or the mask's n_windows is out of range
 * (fwa2_validate names the field);
 * SIZE_MAX for sizes no device can hold (heads * n^2 beyond 2^44 or
 * bw * heads * n^2 beyond 2^52), which fwa2_validate then reports as a
 * workspace that is too small.
 * The figure grows with the device's compute-unit count (one partial dbias
 * tile per persistent workgroup); see fwa2_validate.
 */
size_t fwa2_backward_workspace_bytes(const fwa2_problem* p);

/*
 * o, lse = attention(q, k, v, logit_scale, bias, mask).
 * Replaces _flash_attn_forward (attn_kernel_forward.py:261-345).
 */
int fwa2_forward(const fwa2_problem* p);

/*
 * dq, dk, dv, dbias, dscale from d_o and the saved q, k, v, o, lse.
 * Replaces _flash_attn_backward (attn_kernel_backward.py:567-711), including
 * its delta = rowsum(o * do) pre-pass (:6-51), accumulator zero-fill, down-cast
 * copies and the clamp gate on dscale.
 */
int fwa2_backward(const fwa2_problem* p);

/*
 * fwa2_backward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same kernels and results as fwa2_backward, but the scratch lives
 * in a device array of FWA2_STATIC_SCRATCH_BYTES that the library holds on every GPU it is loaded on until the
 * process ends; p->workspace and p->workspace_bytes are ignored.  The call allocates and frees nothing.
 * Has no counterpart in the reference (whose launcher allocates dq_accum, db_accum, dscale_accum and delta with
 * torch on every call, attn_kernel_backward.py:582-626).
 *   - a problem whose fwa2_backward_workspace_bytes() exceeds FWA2_STATIC_SCRATCH_BYTES is refused with
 *     FWA2_ERR_UNSUPPORTED.  The need grows with the batch (one fp32 delta value per query row, except for
 *     windows of 161 to 256 tokens, whose delta never leaves the chip), with the device's compute-unit count
 *     (one N x N fp32 dbias tile per persistent workgroup) and, for windows of 161 to 256 tokens with a mask,
 *     with the number of windows per image (one N x N fp32 table slot per window and head): 3 heads of
 *     256-token windows with a 64-window mask need 112.5 MiB whatever the batch (the reference's benchmark
 *     shape; fits), 76.5 MiB with a 16-window mask, 36 MiB for
 *     64-token windows at 4 096 per call; windows of 576 tokens and more need their fp32 dk / dv partials here
 *     too (0.7 GiB at 256 windows of 6 heads) and do not fit: use fwa2_backward there;
 *   - the device that is current at the call must be the one the tensors and the stream belong to; the address
 *     of that device's copy of the array is looked up on the first call per device (hipGetSymbolAddress, which
 *     may load the code object): make that first call OUTSIDE any stream capture, e.g. one warm-up call before
 *     the capture starts; later calls on the same device only launch kernels;
 *   - the array costs FWA2_STATIC_SCRATCH_BYTES of device memory on every GPU of every process that loads the
 *     library, whether or not this entry point is ever called;
 *   - every call on a GPU shares that GPU's array: calls that may overlap on one GPU (different streams, or
 *     different threads without ordering) race on it.  Calls on one stream are ordered and safe.  Nothing in
 *     the array needs clearing between calls: every kernel writes what a later kernel of the same call reads.
 */
#define FWA2_STATIC_SCRATCH_BYTES ((size_t)128 << 20)
int fwa2_backward_static(const fwa2_problem* p);

/*
 * Relative position bias of a window of wh x ww tokens (N = wh ww) from its table, for the caller of the
 * operator: replaces the gather by relative_position_index, the permute to [H, N, N] and 16 * sigmoid of
 * flash_win_attn_v2/swin_transformer_v2.py:283-287 (the table is the output of the module's cpb_mlp).
 *   table [(2wh-1)(2ww-1), H], bias [H, N, N], both contiguous and of `dtype` (F16 or BF16);
 *   bias[h][q][k] = 16 sigmoid(table[idx(q,k)][h]),
 *   idx(q,k) = (r_q - r_k + wh - 1)(2ww - 1) + (c_q - c_k + ww - 1) with token = r ww + c
 *   (the closed form of the reference's relative_position_index buffer, swin_transformer_v2.py:240-254).
 */
int fwa2_cpb_bias_forward(const void* table, int dtype, int heads, int wh, int ww, void* bias, void* stream);

/*
 * Gradient of the above with respect to the table: dtable[i][h] = 16 s (1 - s) * sum of dbias[h][q][k] over
 * the pairs with idx(q,k) = i, s = sigmoid(table[i][h]); summed in fp32 in a fixed order.  Replaces what
 * autograd derives for swin_transformer_v2.py:283-287 (sigmoid backward, permute, index_put with accumulate).
 *   dbias [H, N, N] contiguous, dtable [(2wh-1)(2ww-1), H] contiguous, both of `dtype`.
 */
int fwa2_cpb_bias_backward(const void* table, const void* dbias, int dtype, int heads, int wh, int ww, void* dtable,
                           void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FWA2_H */
