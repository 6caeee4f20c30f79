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
 *     matching *_workspace_bytes function;
 *   - the library keeps no mutable global state apart from the per-thread last-error string.
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

#ifdef __cplusplus
}
#endif
#endif /* TRITON_AMD_H_ */
