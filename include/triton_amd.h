/*
 * C ABI of the MI355X (gfx950) implementation of the quantized mixture-of-experts hot path of
 * triton-lang/triton's `python/triton_kernels`.
 *
 * Conventions (every entry point):
 *   - returns int32 status: TK_OK, or a TK_ERR_* code with a message available from tk_last_error();
 *     nothing is thrown across the boundary;
 *   - all pointers are device pointers on the current HIP device unless the comment says "host";
 *   - strides are in ELEMENTS of the pointed-to storage type, sizes are element counts;
 *   - no allocation, no synchronisation, no host read of device data: each call only enqueues
 *     kernels on `stream` (a hipStream_t passed as void*), so every call is stream-ordered and can be
 *     recorded into a HIP graph;
 *   - scratch memory is supplied by the caller (`workspace` arguments) with the size returned by the
 *     matching *_workspace_bytes function (tk_route_static, which owns its scratch, is the one exception);
 *   - the library's mutable global state is the per-thread last-error string and write-once caches filled
 *     under a lock or atomically (the compute-unit count per device, which kernels had their LDS limit raised,
 *     the device address of tk_route_static's scratch array).
 *
 * Each entry point names the reference launch site it replaces; paths are relative to the reference
 * tree root, `python/triton_kernels/triton_kernels/` abbreviated as `tk/`.
 */
#ifndef TRITON_AMD_H_
#define TRITON_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tk_stream_t; /* hipStream_t */

enum tk_status {
  TK_OK = 0,
  TK_ERR_INVALID = 1,     /* bad argument (maps to ValueError) */
  TK_ERR_UNSUPPORTED = 2, /* valid in the reference, not implemented here (NotImplementedError) */
  TK_ERR_LAUNCH = 3       /* HIP reported a launch error (RuntimeError) */
};

enum tk_dtype {
  TK_F32 = 0,
  TK_BF16 = 1,
  TK_F16 = 2,
  TK_E4M3 = 3,  /* OCP float8 e4m3fn */
  TK_E5M2 = 4,  /* OCP float8 e5m2 */
  TK_E2M1 = 5,  /* OCP float4 e2m1, two per byte, even index in the low nibble */
  TK_U8 = 6,
  TK_I16 = 7,
  TK_I32 = 8
};

enum tk_mx_rounding {
  TK_MX_ROUND_UP = 0,  /* scale = 2^ceil(log2(max/max_q)) */
  TK_MX_ROUND_DOWN = 1 /* scale = 2^floor(log2(max/max_pow2_q)) */
};

/* Library version (major*10000 + minor*100 + patch). */
int32_t tk_version(void);

/* Message of the last error raised on the calling thread ("" if none).  Host pointer. */
const char* tk_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * MX (microscaling) quantise / dequantise
 * ---------------------------------------------------------------------------------------------- */

/*
 * Replaces the `_downcast_to_mxfp[(blocks_out_dim, blocks_quant_dim)](...)` launch of
 * tk/numerics_details/mxfp.py:77-86 (kernel tk/numerics_details/mxfp_details/_downcast_to_mxfp.py:149-215).
 *
 * The source is viewed as [outer, axis_len, inner] with the given element strides and is read in
 * place (no transposed temporary).  Quantisation runs along `axis_len` in blocks of 32
 * (axis_len % 32 == 0).  Outputs are dense with the quantised axis innermost:
 *   out_vals   [outer, inner, axis_len/2] uint8 (TK_E2M1)  or [outer, inner, axis_len] (TK_E4M3/TK_E5M2)
 *   out_scales [outer, inner, axis_len/32] uint8 (e8m0 exponent bytes)
 * `inner` is the product mid x inner_last of the source dimensions after the axis (inner_last = the
 * last one, fastest in the source); output lines are ordered (outer, last, mid), i.e. the order of
 * `x.transpose(axis, -1)`, which is the storage order `StridedLayout(major_dim=axis)` gives the
 * reference's outputs (tk/numerics_details/mxfp.py:61-64).  For axis == ndim-2 this is plain
 * [outer, inner, axis].  Supported source layouts: stride_inner == 1, or
 * stride_axis == 1 with inner == 1.  src_dtype in {TK_F32, TK_BF16, TK_F16}.
 */
int32_t tk_mx_downcast(const void* src, int32_t src_dtype, int64_t outer, int64_t axis_len, int64_t inner,
                       int64_t inner_last, int64_t stride_outer, int64_t stride_axis, int64_t stride_inner, void* out_vals,
                       void* out_scales, int32_t out_kind, int32_t rounding, tk_stream_t stream);

/*
 * Replaces the `_upcast_from_mxfp[(blocks_out_dim, blocks_quant_dim)](...)` launch of
 * tk/numerics_details/mxfp.py:157-167 (kernel tk/numerics_details/mxfp_details/_upcast_from_mxfp.py:109-220)
 * together with the two transposed copies around it (mxfp.py:122-123,172).
 *
 * Inputs are dense with the quantised axis innermost (the layout tk_mx_downcast writes):
 *   vals [outer, inner, axis_len/2 or axis_len], scales [outer, inner, axis_len/32], lines ordered
 *   (outer, last, mid) as above.
 * The output is written through the given element strides of its [outer, axis_len, inner] view;
 * supported: ostride_inner == 1, or ostride_axis == 1 with inner == 1.  out_dtype in
 * {TK_F32, TK_BF16, TK_F16}.  Value = element * 2^(scale-127) in fp32, clamped to the finite range of
 * out_dtype, then rounded to nearest even.
 */
int32_t tk_mx_upcast(const void* vals, const void* scales, int32_t kind, int64_t outer, int64_t axis_len,
                     int64_t inner, int64_t inner_last, void* out, int32_t out_dtype, int64_t ostride_outer, int64_t ostride_axis,
                     int64_t ostride_inner, tk_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Router: top-k (+softmax), expert histogram, gather/scatter permutations, ragged block schedule
 * ---------------------------------------------------------------------------------------------- */

/*
 * One routing pass.  Replaces, in three launches, the reference's
 *   `_topk_forward[(pids,)](...)`                          tk/topk.py:59-67
 *   `_sum_bitmatrix_rows[(grid_m, grid_n)](...)`           tk/tensor_details/bitmatrix_details/sum_bitmatrix_rows.py:89-97
 *   `_bitmatrix_metadata_compute_stage1/2[...]`            tk/tensor_details/bitmatrix.py:128-145
 *   `_ragged_tensor_metadata_memset/compute[...]`          tk/tensor_details/ragged_tensor.py:197-208
 * and the torch glue `gather = col_sorted // k`, `gammas = vals.flatten()[col_sorted]`
 * (python/triton_kernels/tests/test_distributed.py:203-210).
 *
 * Selection is a stable descending sort: ties go to the lower expert id; outputs are ordered by value,
 * largest first; the softmax runs over the k kept logits in fp32.  Rows >= n_rows are left untouched
 * in vals / indx / bitmatrix and are not routed.  Optional outputs may be NULL; when col_sum is NULL
 * only the top-k step runs.  Limits of the entry point: n_experts <= 2048, k <= min(64, n_experts) (the
 * reference's `topk` is narrower in k: a power of two <= 32, which the Python host enforces).
 */
typedef struct tk_route_desc {
  const void* logits; /* [n_tokens, n_experts], unit stride along experts; may be NULL with use_provided_indx */
  int32_t logits_dtype; /* TK_F32, TK_BF16, TK_F16 */
  int64_t logits_stride_m;
  int32_t n_tokens;
  int32_t n_rows;            /* rows to route, -1 = all */
  const int32_t* n_rows_ptr; /* device scalar overriding n_rows, or NULL */
  int32_t n_experts;
  int32_t k;
  int32_t apply_softmax;
  int32_t use_provided_indx; /* 1: `indx` is an input (tk/topk.py:121-123) */
  void* vals;                /* out [n_tokens, k], logits dtype, or NULL */
  void* indx;                /* [n_tokens, k] */
  int32_t indx_dtype;        /* TK_I16 */
  void* bitmatrix;           /* out uint32 [ceil(E/32)][bitmatrix_stride_w]: word w of token t at w*stride + t; or NULL */
  int64_t bitmatrix_stride_w;
  int32_t* col_sum;         /* out [n_experts] tokens per expert */
  int32_t* col_sorted_indx; /* out [n_tokens*k] flat position t*k+j of each expert-sorted row, -1 padded */
  int32_t* row_sorted_indx; /* out [n_tokens*k] inverse permutation, -1 padded */
  int32_t* gather_indx;     /* out [n_tokens*k] token of each expert-sorted row (= col_sorted / k), or NULL */
  void* gammas;             /* out [n_tokens*k] gate value of each expert-sorted row (logits dtype), or NULL */
  /* ragged metadata of col_sum for block sizes 16, 32, 64, 128, 256 (all NULL to skip) */
  int32_t* slice_offs;     /* out [n_experts + 1] */
  int32_t* block_offs;     /* out [5][block_offs_stride], first n_experts + 1 entries of each row */
  int64_t block_offs_stride;
  int32_t* block_schedule; /* out [5][block_schedule_stride], first max_n_blocks entries of each row */
  int64_t block_schedule_stride;
  int32_t max_n_blocks;
  void* workspace; /* tk_route_workspace_bytes(n_tokens, n_experts) bytes, needed when col_sum != NULL */
} tk_route_desc;

int64_t tk_route_workspace_bytes(int32_t n_tokens, int32_t n_experts);
int32_t tk_route(const tk_route_desc* desc, tk_stream_t stream);

/*
 * tk_route for callers that cannot allocate.  No counterpart in the reference: it is for code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc, which cannot provide `workspace`.  Same
 * arguments and results as tk_route, except that `desc->workspace` is ignored: the kernels' scratch memory is a
 * device array inside the library (TK_ROUTE_STATIC_SCRATCH_BYTES per GPU, held until the process ends), so the
 * call allocates nothing.  Problems with tk_route_workspace_bytes(n_tokens, n_experts) above that size are
 * refused with TK_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (different streams, different threads) race and must be serialised by the caller; calls in stream order are
 * safe, the array's previous contents are never read.
 * The array's device address is looked up once per device (hipGetSymbolAddress, which may load the code object):
 * by tk_route_static_prepare(), or else by the first tk_route_static call on that device.  That lookup must not
 * happen while a stream is capturing, so code that captures tk_route_static calls tk_route_static_prepare() (or
 * makes one eager tk_route_static call) on each device beforehand.  Device ids 0..63 are served; others are
 * refused with TK_ERR_UNSUPPORTED.
 */
#define TK_ROUTE_STATIC_SCRATCH_BYTES (2 * 1024 * 1024)
int32_t tk_route_static(const tk_route_desc* desc, tk_stream_t stream);
/* Set-up of tk_route_static on the current device (no device work, allocates nothing; safe to call repeatedly). */
int32_t tk_route_static_prepare(void);

/*
 * Replaces `_topk_backward` (tk/topk_details/_topk_backward.py:5-51, launched by tk/topk.py:76-85): gradient of the
 * kept logits' softmax (or of the plain selection) scattered back into dx [n_tokens, n_experts]; every other element
 * of dx, and every row >= n_rows, is zero.  x, dy, dx share `dtype` (fp32 / bf16 / fp16); strides in elements.
 */
int32_t tk_topk_backward(const void* x, int32_t dtype, int64_t stride_xm, const int16_t* indx, int64_t stride_im, const void* dy,
                         int64_t stride_dym, void* dx, int64_t stride_dxm, int32_t n_tokens, int32_t n_experts, int32_t k,
                         int32_t apply_softmax, int32_t n_rows, const int32_t* n_rows_ptr, tk_stream_t stream);

/*
 * Replaces `_ragged_tensor_metadata_memset` + `_ragged_tensor_metadata_compute`
 * (tk/tensor_details/ragged_tensor.py:183-210): slice_offs = [0] + cumsum(slice_sizes); for block sizes
 * 16..256: block_offs = [0] + cumsum(ceil(slice_sizes / bs)) and block_schedule[offs[s] + b] =
 * (b << 16) | s, padded with -1 up to max_n_blocks.
 */
int32_t tk_ragged_metadata(const int32_t* slice_sizes, int32_t n_slices, int32_t* slice_offs, int32_t* block_offs,
                           int64_t block_offs_stride, int32_t* block_schedule, int64_t block_schedule_stride,
                           int32_t max_n_blocks, tk_stream_t stream);

/*
 * Replaces `_remap_ragged_tensor_metadata` (tk/tensor_details/ragged_tensor.py:309-381): metadata of the ragged
 * tensor that keeps the slices with slice_map[slice] != -1, in their order.  Kept slice sizes, slice offsets and
 * block offsets are compacted to the front (their values unchanged) and followed by -1; schedule entries of kept
 * slices are compacted and carry slice_map[slice] as their slice id; block_offs_out[b][number of kept slices]
 * receives the number of schedule entries kept.  Inputs and outputs have the shapes of tk_ragged_metadata's.
 */
int32_t tk_ragged_remap(const int32_t* slice_sizes, const int32_t* slice_offs, const int32_t* block_offs,
                        int64_t block_offs_stride, const int32_t* block_schedule, int64_t block_schedule_stride,
                        const int32_t* slice_map, int32_t n_slices, int32_t n_block_sizes, int32_t max_n_blocks,
                        int32_t* slice_sizes_out, int32_t* slice_offs_out, int32_t* block_offs_out,
                        int64_t block_offs_out_stride, int32_t* block_schedule_out, int64_t block_schedule_out_stride,
                        tk_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Ragged expert GEMM
 * ---------------------------------------------------------------------------------------------- */

/*
 * How `w` / `w_mx_scale` are laid out.  TK_W_STRIDED is the reference's strided form (what
 * `downcast_to_mxfp(w, uint8, axis=1)` returns, tk/numerics_details/mxfp.py:61-64).  TK_W_TILED is this
 * library's pre-tiled MXFP4 form, the counterpart of the reference's architecture-specific weight layouts
 * (tk/tensor_details/layout.py:26-54, built once per model with `convert_layout`): per expert, per fragment
 * F of 32 output columns (N padded to 32), per K-stage s of 128 (K padded to 128, zero weights):
 *   values  one 2048-byte block at ((F * S + s) * 2048), S = ceil(K / 128), ordered [q:2][lane:64][16 bytes];
 *           lane = h*32 + c holds the packed e2m1 bytes (even k in the low nibble) of column F*32 + c for
 *           k in [s*128 + h*64 + q*32, +32);
 *   scales  one 128-byte block at ((F * S + s) * 128) ordered [c:32][4]: the four e8m0 bytes of column
 *           F*32 + c for the stage's four 32-element blocks.
 * With this layout and block_m >= 64: at most 1024 slices; x and y each span less than 4 GiB / 2 GiB; output rows are
 * 16-byte aligned with a row stride of at least N_out rounded up to 8 (whole 16-byte pieces are written, the
 * padding columns receive unspecified values); x_row_scale / w_col_scale are not supported.
 * With w_dtype == TK_E4M3 (e4m3 activations, no MX scales) TK_W_TILED is the one-byte variant of the same idea:
 *   values  K padded to 256 (S = 2 * ceil(K / 256) blocks of 128 per fragment); one 4096-byte block at
 *           ((F * S + s) * 4096) ordered [q:4][lane:64][16 bytes]; lane = h*32 + c holds
 *           the e4m3 bytes of column F*32 + c for k in [s*128 + (q/2)*64 + h*32 + (q%2)*16, +16);
 *           block_m must be 128 or 256.
 * The w_stride_e / ws_stride_e fields give the bytes from one expert to the next; the k / n strides are unused.
 */
enum tk_w_layout { TK_W_STRIDED = 0, TK_W_TILED = 1 };

enum tk_activation {
  TK_ACT_NONE = 0,
  TK_ACT_SWIGLU = 1 /* interleaved (gate, linear) columns -> N/2 outputs, tk/swiglu_details/_swiglu.py:55-70 */
};

/*
 * Operands of one ragged GEMM launch.  Plain data, filled by the host; pointers are device pointers,
 * NULL means "absent".  Mirrors the argument list of the `_matmul[(grid,)](...)` launch of
 * tk/matmul.py:659-726 restricted to what a mixture-of-experts forward uses.
 *
 *   Y[dst(r), :] = act( (X[src(r), :] @ W[e(r)]) * x_row_scale[src(r)] * w_col_scale[e(r), :]
 *                        + bias[e(r), :] ) * gammas[r]
 *
 * r runs over rows in expert-sorted order; e(r) is the slice containing r; src(r) = gather_indx[r]
 * (or r); dst(r) = scatter_indx[r] (or r), rows with dst(r) == -1 are not written.  Accumulation is
 * fp32; the epilogue order is that of tk/matmul_details/_matmul.py:507-559.
 */
typedef struct tk_gemm_desc {
  /* activations: [rows, K], unit stride along K */
  const void* x;
  int32_t x_dtype; /* TK_BF16, TK_F16 (with TK_F16 weights and output), TK_E4M3 with x_row_scale (plain fp8), or TK_E4M3
                    * with x_mx_scale (MXFP8) */
  int64_t x_stride_m;
  const float* x_row_scale; /* fp32 per row of x, read at the source row src(r), or NULL */
  /* weights: [E, K, N]; e2m1 is packed two per byte along K and the strides count bytes */
  const void* w;
  int32_t w_dtype; /* TK_BF16, TK_F16 (strided layout only), TK_E2M1 (needs w_mx_scale), TK_E4M3 */
  int64_t w_stride_e, w_stride_k, w_stride_n;
  const void* w_mx_scale; /* uint8 e8m0 [E, K/32, N] or NULL */
  int64_t ws_stride_e, ws_stride_k, ws_stride_n;
  const float* w_col_scale; /* fp32 [E, N] (unit stride along N) or NULL */
  int64_t wcs_stride_e;
  /* bias [E, N] (unit stride along N), fp32 or bf16 */
  const void* bias;
  int32_t bias_dtype;
  int64_t bias_stride_e;
  /* row indirection and per-row scale (expert-sorted order) */
  const int32_t* gather_indx;
  const int32_t* scatter_indx;
  int32_t scatter_len;
  const void* gammas;
  int32_t gammas_dtype; /* TK_F32 or TK_BF16 */
  /* ragged metadata for `block_m` (tk/tensor_details/ragged_tensor.py:12-94); all NULL = one slice of M rows */
  const int32_t* slice_sizes;
  const int32_t* slice_offs;
  const int32_t* block_offs;     /* [n_slices + 1] for block_m */
  const int32_t* block_schedule; /* [grid_m] for block_m, (block << 16) | slice, -1 padded */
  int32_t n_slices;
  int32_t block_m; /* 16, 32, 64 or 128; tiled MXFP4 weights also 256; tiled e4m3 weights 128 or 256 only */
  int32_t grid_m;  /* number of row blocks to launch (an upper bound in ragged mode) */
  int32_t M, N, K; /* M: rows of the single slice when not ragged; N: columns of W; K: reduction */
  /* output [rows, N or N/2], unit stride along N */
  void* y;
  int32_t y_dtype; /* TK_BF16, TK_F16 (fp16 operands), or with y_mx_scale TK_E4M3 / TK_E5M2 / TK_E2M1 (see there) */
  int64_t y_stride_m;
  int32_t activation; /* enum tk_activation */
  float act_alpha, act_limit;
  int32_t act_has_limit;
  int32_t w_layout; /* enum tk_w_layout */
  /* compute units to leave idle: the persistent kernels (tiled weight layouts, block_m >= 64) launch that many
   * workgroup slots fewer (the reference's `idle_sms`, tk/matmul_details/opt_flags.py:525-529); 0 = use all */
  int32_t idle_cus;
  /* Optional scratch for the persistent kernels: TK_GEMM_TILE_COUNTER_WORDS int32 words, zero before the first
   * launch that uses them.  With it, and when the tiles do not divide evenly among the workgroups, a workgroup
   * takes its first two tiles from a fixed schedule and claims the following ones with atomic counters (one queue
   * per XCD), which evens out tiles of different cost; the kernel leaves the words zero again, so one buffer serves
   * any number of launches in stream order, but launches that may overlap in time (other streams) need their own
   * words.  NULL = fixed schedule.  No counterpart in the reference (its AMD path is not persistent). */
  int32_t* tile_counters;
  /* rows of x (with gather_indx: every index is below it); 0 = not stated (then M when not gathering).  The kernels
   * for tiled MXFP4 weights at block_m >= 64 need x to span less than 4 GiB and refuse larger ones; with
   * gather_indx they refuse a descriptor that leaves x_rows at 0 (TK_ERR_INVALID). */
  int64_t x_rows;
  /* MXFP8 activations (x_dtype TK_E4M3): e8m0 block scales uint8 [rows of x, K / 32], unit stride along K, one per
   * 32 consecutive k of a row (tk/matmul.py:130-132 `a_mx_scale`); NULL = x is not MX-quantised.  Goes with tiled
   * MXFP4 weights, block_m 128 or 256, and runs on v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in their
   * storage formats. */
  const void* x_mx_scale;
  int64_t xs_stride_m;
  /* MX-quantised output: the epilogue quantises the fp32 accumulator, after bias, activation and gate weight, in blocks
   * of 32 output columns (the `QUANTIZE_MXFP8` / `QUANTIZE_MXFP4` epilogues, tk/matmul_details/_matmul.py:593-637):
   * values to y, one e8m0 byte per block (round-up rule) to y_mx_scale [rows of y, N_out / 32]; N_out % 32 == 0.
   *   MXFP8 activations (x_mx_scale):                                 y_dtype TK_E4M3
   *   bf16 activations, tiled MXFP4 weights, block_m 128 or 256:      y_dtype TK_E4M3, TK_E5M2 or TK_E2M1 (two codes per byte,
   *     even column in the low nibble; y_stride_m then counts bytes); rows of y 8-byte aligned; not with betas /
   *     out_alpha / acc_in or the fused combine
   * NULL = plain bf16 output.  Other operand combinations quantise in a second pass (tk_mx_downcast on the bf16 result). */
  void* y_mx_scale;
  int64_t ys_stride_m;
  /* Fused top-k combine behind the scatter (bf16 activations, tiled MXFP4 weights, no activation).  At block_m >= 64
   * the persistent kernel sums when all its workgroups have written their tiles (a device-wide arrival count in words
   * 9..31 of tile_counters, which must be given; word 11 is raised, and stays, if a bounded wait for the other
   * workgroups runs out; combine_counters is not used; N % 8 == 0, 16-byte aligned rows of combine_out, and the
   * launch must not share the GPU with another launch that waits for its own workgroups).  At block_m 16 or 32:
   * scatter_indx maps expert-sorted row r to flat position t * combine_k + j; besides y [tokens * combine_k, N] the
   * kernel writes combine_out[t, :] = sum over j of y[t * combine_k + j, :] (fp32 sum in j order, bf16 result: what
   * tk_reduce_mid computes from y), by the wave that completes token t's rows last.  combine_counters:
   * tokens * ceil(N / 32) zeroed int32 words; a launch leaves them zero again PROVIDED every token has exactly
   * combine_k routed rows.  A token with fewer (dropped entries, rows of experts that live on another rank) never
   * completes: its row of combine_out is not written and its counter words stay non-zero, which corrupts that
   * token in every later launch that shares the words, so callers must not request the combine for such routing
   * (or must clear the words themselves, with a fill kernel on the same stream).  The Python host keeps one buffer
   * of 65536 words per (device, stream) and falls back to the separate tk_reduce_mid launch when
   * tokens * ceil(N / 32) exceeds it (728 tokens at N = 2880).  0 = no combine.  Replaces the separate
   * `reduce(y.view(T, k, -1), dim=1)` launch of tk/reduce.py:1143-1165 after the scatter of
   * tk/matmul_details/_matmul.py:535-569. */
  int32_t combine_k;
  void* combine_out; /* bf16 [tokens, N], unit stride along N */
  int64_t combine_stride_m;
  int32_t* combine_counters;
  /* Less common options of the reference's epilogue, in its order (tk/matmul_details/_matmul.py:547-559,581-591):
   *   acc = acc * scales + bias * betas[r];  acc *= out_alpha;  out = act(acc) * gammas[r];  out += acc_in[row, :]
   * betas: per expert-sorted row, fp32 or bf16 (`betas`, tk/matmul.py:251); out_alpha: scalar, applied when
   * has_out_alpha != 0 (tk/matmul.py:253); acc_in: a tensor of the output's shape and type that is added to the
   * result (`c_acc_in`, tk/matmul.py:258,529-535; not together with scatter_indx).  Served by the kernels with the
   * shared epilogue: strided weights, tiled e4m3 weights, tiled MXFP4 weights at block_m 16 / 32 without the fused
   * combine, and MXFP8 activations without an MX output; any other combination is refused with TK_ERR_UNSUPPORTED. */
  const void* betas;
  int32_t betas_dtype;
  int32_t has_out_alpha;
  float out_alpha;
  const void* acc_in;
  int64_t acc_in_stride_m;
} tk_gemm_desc;

#define TK_GEMM_TILE_COUNTER_WORDS 32

/* Replaces the `_matmul[(grid,)](...)` launch of tk/matmul.py:659-726 (kernel tk/matmul_details/_matmul.py:43-672). */
int32_t tk_moe_gemm(const tk_gemm_desc* desc, tk_stream_t stream);

/*
 * GEMM with a ragged REDUCTION dimension (the expert weight gradient): for every slice e
 *   y[e, m, n] = sum over k < slice_sizes[e] of a[m, a_slice_offs[e] + k] * b[b_slice_offs[e] + k, n]
 * Replaces the `_matmul` launch of tk/matmul.py:659-726 when `b_ragged_metadata` is given (tk/matmul.py:376-384:
 * ragged_dimension "K", batch = number of slices; kernel side tk/matmul_details/_matmul.py:252-272; torch statement
 * tk/matmul.py:852-875).  The two operands carry their own slice offsets (one of them may be padded per slice); the
 * sizes are those of b's metadata.  An empty slice yields a zero matrix.  No bias, gather, scatter or scales.
 * a, b: TK_BF16 or TK_F16 (same type), any strides (in elements); fastest when the reduction index is the slow
 * dimension of both (a = x^T, b = dy) with 16-byte aligned bases and strides that are multiples of 8.
 * y: [n_slices, M, N], unit stride along N, TK_BF16 / TK_F16 / TK_F32; fp32 accumulation.
 */
typedef struct tk_ragged_k_desc {
  const void* a;
  int32_t dtype; /* of a and b */
  int64_t a_stride_m, a_stride_k;
  const void* b;
  int64_t b_stride_k, b_stride_n;
  void* y;
  int32_t y_dtype;
  int64_t y_stride_e, y_stride_m;
  int32_t M, N, n_slices;
  const int32_t* slice_sizes;  /* [n_slices] reduction length per slice */
  const int32_t* a_slice_offs; /* [n_slices] first k of the slice in a */
  const int32_t* b_slice_offs; /* [n_slices] first k of the slice in b */
  /* extent of the reduction dimension of a and of b (a is [M, a_k_extent], b is [b_k_extent, N]); every slice lies
   * inside.  0 = not stated: the kernel then cannot bound its loads by the tensors' ends and takes its general path. */
  int64_t a_k_extent, b_k_extent;
} tk_ragged_k_desc;

int32_t tk_ragged_k_gemm(const tk_ragged_k_desc* desc, tk_stream_t stream);

/*
 * A whole decode-sized MoE FFN layer in ONE launch:
 *   out[t, :] = sum over j < k of gate[t, j] * ( swiglu( x[t, :] @ W1[e] + b1[e] ) @ W2[e] + b2[e] ),  e = indx[t, j]
 * with (indx, gate) = top-k (+softmax) of logits[t, :] exactly as tk_route selects them.  Replaces, for
 * n_tokens * k <= TK_DECODE_MAX_ROWS, the sequence the reference's MoE block issues (python/triton_kernels/bench/
 * bench_mlp.py:72-79 and tests/test_distributed.py:203-220): `topk` + metadata launches (tk/topk.py:59-67,
 * tk/tensor_details/bitmatrix.py:128-145, tk/tensor_details/ragged_tensor.py:197-208), two `_matmul` launches
 * (tk/matmul.py:659-726: gather + fused swiglu, then scatter + gammas) and `reduce` over the k rows of a token
 * (tk/reduce.py:1143-1165).  Same arithmetic as that sequence on this library's kernels: bf16 MFMA with fp32
 * accumulation on MXFP4 weights expanded in registers, swiglu on the fp32 accumulator, the hidden activations and the
 * k partial rows rounded to bf16, the combine summed in fp32 in j order.
 *
 * W1 [E, d_model, 2*d_ff] and W2 [E, d_ff, d_model] are MXFP4 in the tiled layout (TK_W_TILED) with tiled scales;
 * x is bf16 [n_tokens, d_model]; biases bf16 or fp32 [E, N] or NULL; out bf16 [n_tokens, d_model].
 * Limits: n_tokens * k <= TK_DECODE_MAX_ROWS, n_experts <= TK_DECODE_MAX_EXPERTS, d_model and d_ff <= 3072 and
 * multiples of 8; otherwise TK_ERR_UNSUPPORTED (callers then take tk_route + tk_moe_gemm).
 *
 * The kernel is persistent: its workgroups must all be resident together (the grid is sized from the occupancy the
 * runtime reports) because workgroups of the second GEMM wait for the first GEMM's rows of other workgroups.  Two
 * launches of it that overlap in time on one device (different streams) could each hold part of the GPU and wait
 * for the rest; callers serialise them.  Every wait is bounded by `spin_limit` polls (0 = default, about a second):
 * a wait that runs out sets bit 0 of the error word and the launch finishes with a wrong result instead of hanging.
 *
 * workspace: tk_moe_decode_layer_workspace_bytes(...) bytes, 256-byte aligned: the hidden activations, the k partial
 * rows and, at its end, the synchronisation words: [0] finished workgroups, [1] error word (sticky; 0 = fine),
 * then the counters.  The words must be ZERO before the first launch; a launch leaves them zero (except a raised
 * error word), so launches in stream order share one workspace.  indx_out / vals_out: optional [n_tokens, k]
 * int16 / fp32 copies of the routing decision.
 */
#define TK_DECODE_MAX_ROWS 256
#define TK_DECODE_MAX_EXPERTS 512
typedef struct tk_decode_layer_desc {
  const void* x; /* bf16 [n_tokens, d_model], unit stride along d_model, 16-byte aligned */
  int64_t x_stride_m; /* elements; >= d_model, a multiple of 8, all rows within 2 GiB of x */
  const void* logits; /* [n_tokens, n_experts], TK_F32 or TK_BF16 */
  int32_t logits_dtype;
  int64_t logits_stride_m;
  int32_t n_tokens, n_experts, k, apply_softmax;
  int32_t d_model, d_ff;
  const void* w1; /* tiled MXFP4 [E, d_model, 2*d_ff] */
  const void* w1_mx_scale;
  int64_t w1_stride_e, w1s_stride_e; /* bytes */
  const void* b1;                    /* [E, 2*d_ff] or NULL */
  int32_t b1_dtype;
  int64_t b1_stride_e;
  const void* w2; /* tiled MXFP4 [E, d_ff, d_model] */
  const void* w2_mx_scale;
  int64_t w2_stride_e, w2s_stride_e;
  const void* b2; /* [E, d_model] or NULL */
  int32_t b2_dtype;
  int64_t b2_stride_e;
  float act_alpha, act_limit; /* swiglu */
  int32_t act_has_limit;
  void* out; /* bf16 [n_tokens, d_model] */
  int64_t out_stride_m;
  void* indx_out;   /* optional int16 [n_tokens, k] */
  float* vals_out;  /* optional fp32 [n_tokens, k] */
  void* workspace;
  int32_t spin_limit;
} tk_decode_layer_desc;

int64_t tk_moe_decode_layer_workspace_bytes(int32_t n_tokens, int32_t k, int32_t n_experts, int32_t d_ff, int32_t d_model);
int32_t tk_moe_decode_layer(const tk_decode_layer_desc* desc, tk_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Element-wise companions of the GEMM
 * ---------------------------------------------------------------------------------------------- */

/*
 * Standalone swiglu; replaces the `_swiglu[grid](...)` launch of tk/swiglu.py:56-79.
 * a [M, 2*n_out] with interleaved (gate, linear) columns -> out [M, n_out], same dtype
 * (TK_BF16 / TK_F16 / TK_F32), fp32 arithmetic.  n_rows_ptr (device scalar, may be NULL) bounds M.
 */
int32_t tk_swiglu(const void* a, int32_t dtype, int64_t M, int64_t n_out, int64_t stride_am, void* out,
                  int64_t stride_om, float alpha, float limit, int32_t has_limit, const int32_t* n_rows_ptr,
                  tk_stream_t stream);

/*
 * Sum over the middle dimension; replaces the `_reduce_forward[grid](...)` launch of tk/reduce.py:664-853
 * for dim == 1 (the k-way combine of expert outputs).
 * y[a, c] = sum_j (mask[a, j, c] ? x[a, j, c] * scale[a, j, c] : 0); x [A, K, C] with unit stride along C;
 * mask (uint8/bool) and scale (fp32) are optional and addressed through their own strides (0 = broadcast);
 * fp32 accumulation in j order; y has x's dtype.
 */
int32_t tk_reduce_mid(const void* x, int32_t dtype, int64_t A, int64_t K, int64_t C, int64_t sx0, int64_t sx1,
                      const void* mask, int64_t sm0, int64_t sm1, int64_t sm2, const float* scale, int64_t ss0,
                      int64_t ss1, int64_t ss2, void* y, int64_t sy0, tk_stream_t stream);

/*
 * Replaces `_reduce_backward` (tk/reduce.py:859-1049) for the same subset as tk_reduce_mid: dx [A, K, C] contiguous,
 * dx[a, j, c] = mask[a, j, c] ? dy[a, c] * scale[a, j, c] : 0, in dy's dtype.
 */
int32_t tk_reduce_mid_backward(const void* dy, int32_t dtype, int64_t A, int64_t K, int64_t C, int64_t sdy0, const void* mask,
                               int64_t sm0, int64_t sm1, int64_t sm2, const float* scale, int64_t ss0, int64_t ss1, int64_t ss2,
                               void* dx, tk_stream_t stream);

/*
 * Measurement aid (no counterpart in the reference): a kernel of nothing but MFMA instructions on register operands,
 * `n_workgroups` workgroups of four waves.  `kind` 0: `iters` x 8 v_mfma_f32_32x32x16_bf16 per wave (32768 FLOP each);
 * 1: `iters` x 8 v_mfma_f32_32x32x64_f8f6f4 on e4m3 operands (131072 FLOP each); 2: `iters` x 16
 * v_mfma_f32_16x16x32_bf16 (16384 FLOP each).  bench.py times it to report the MFMA rates this board sustains under
 * its power cap.  `out`: at least n_workgroups * 256 floats of device memory (practically never written).
 */
int32_t tk_probe_mfma(float* out, int32_t n_workgroups, int32_t iters, int32_t kind, tk_stream_t stream);

/*
 * Per-row dynamic quantisation of bf16 activations to OCP e4m3: scales[m] = amax_m / 448 (1 for a zero
 * row), q[m, :] = saturating_cast(x[m, :] / scales[m]).  No counterpart kernel in the reference: its
 * benchmark casts activations to fp8 with a plain torch `.to()` (python/triton_kernels/bench/bench_mlp.py:169);
 * the scales feed tk_gemm_desc.x_row_scale.
 */
int32_t tk_quant_fp8_rows(const void* x, int32_t dtype, int64_t M, int64_t K, int64_t stride_m, void* q,
                          int64_t stride_qm, float* scales, tk_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Host check hooks (no device work, no GPU needed)
 * ---------------------------------------------------------------------------------------------- */

/*
 * The scalar conversions the MX kernels use, evaluated on the host so that their bit-exactness can be tested on
 * a machine without a GPU.  tk_host_mx_convert: out[i] = code of in[i] in `kind` (TK_E2M1: 4-bit code in the low
 * nibble; TK_E4M3 / TK_E5M2: the byte), round to nearest even with saturation.  tk_host_mx_scale: out[i] = e8m0
 * byte of the block scale for a block whose largest magnitude is absmax[i] (tk/numerics_details/mxfp.py:251-290).
 * Host pointers.
 */
int32_t tk_host_mx_convert(const float* in, int64_t n, int32_t kind, uint8_t* out);
int32_t tk_host_mx_scale(const float* absmax, int64_t n, int32_t kind, int32_t rounding, uint8_t* out);

#ifdef __cplusplus
}
#endif
#endif /* TRITON_AMD_H_ */
