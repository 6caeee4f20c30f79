// C-ABI entry of the ragged (grouped) expert GEMM with fused gather, MX dequantisation, bias, swiglu, gate scaling
// and scatter:
//
//   Y[dst(r), :] = act( (X[src(r), :] @ W[e(r)]) * sx[src(r)] * sw[e(r), :] + bias[e(r), :] ) * gamma[r]
//
// validates the descriptor and hands it to one kernel family (moe_gemm_strided / _mxn / _mxd / _f8n / _mx8n .hip).
#include "gemm_common.h"

using namespace tk;

extern "C" int32_t tk_moe_gemm(const tk_gemm_desc* d, tk_stream_t stream) {
  if (!d) return fail(TK_ERR_INVALID, "tk_moe_gemm: null descriptor");
  if (d->M < 0 || d->N < 0 || d->K < 0) return fail(TK_ERR_INVALID, "tk_moe_gemm: negative size");
  if (d->M == 0 || d->N == 0 || d->grid_m == 0) return TK_OK;
  if (!d->x || !d->w || !d->y) return fail(TK_ERR_INVALID, "tk_moe_gemm: null operand");
  const bool f16 = d->x_dtype == TK_F16 || d->w_dtype == TK_F16;  // fp16 x fp16 -> fp16, strided weights only
  if (f16 && (d->x_dtype != TK_F16 || d->w_dtype != TK_F16 || d->y_dtype != TK_F16 || d->w_layout != TK_W_STRIDED || d->tile_counters || d->combine_counters))
    return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: fp16 activations go with strided fp16 weights and an fp16 output");
  if (d->x_dtype != TK_BF16 && d->x_dtype != TK_E4M3 && !f16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activations must be bf16, fp16 or e4m3 (dtype %d)", d->x_dtype);
  const bool mx_act = d->x_dtype == TK_E4M3 && d->x_mx_scale != nullptr;  // MXFP8 activations: scaled-MFMA path
  if (!mx_act && (d->x_dtype == TK_E4M3) != (d->w_dtype == TK_E4M3)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: e4m3 activations go with e4m3 weights, or with MX scales and tiled MXFP4 weights (x dtype %d, w dtype %d)", d->x_dtype, d->w_dtype);
  // MX-quantised output from the fp32 accumulator: e4m3 on the MXFP8-activation path; e4m3 / e5m2 / packed e2m1 with bf16
  // activations and tiled MXFP4 weights at block_m 128 / 256
  const bool mx_out = d->y_mx_scale != nullptr && (d->y_dtype == TK_E4M3 || (!mx_act && (d->y_dtype == TK_E5M2 || d->y_dtype == TK_E2M1)));
  const bool mx_out_bf16 = mx_out && !mx_act && d->x_dtype == TK_BF16 && d->w_layout == TK_W_TILED && d->w_dtype == TK_E2M1 && (d->block_m == 128 || d->block_m == 256);
  if (d->y_dtype != TK_BF16 && !f16 && !(mx_out && (mx_act || mx_out_bf16)))
    return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: output must be bf16, or MX-quantised (y_mx_scale): e4m3 with MXFP8 activations; e4m3, e5m2 or e2m1 with bf16 activations and tiled MXFP4 weights at block_m 128 / 256 (dtype %d)", d->y_dtype);
  if (d->activation != TK_ACT_NONE && d->activation != TK_ACT_SWIGLU) return fail(TK_ERR_INVALID, "tk_moe_gemm: bad activation %d", d->activation);
  if (d->activation == TK_ACT_SWIGLU && d->N % 2) return fail(TK_ERR_INVALID, "tk_moe_gemm: swiglu needs an even N");
  const int xe = d->x_dtype == TK_E4M3 ? 16 : 8;  // elements per 16 bytes
  if (d->K % xe) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: K must be a multiple of %d (got %d)", xe, d->K);
  if (d->x_stride_m % xe || (reinterpret_cast<uintptr_t>(d->x) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activation rows must be 16-byte aligned");
  if (d->slice_sizes && (!d->slice_offs || !d->block_offs || !d->block_schedule)) return fail(TK_ERR_INVALID, "tk_moe_gemm: incomplete ragged metadata");
  if (d->n_slices >= 65536) return fail(TK_ERR_INVALID, "tk_moe_gemm: at most 65535 slices");
  GemmParams p;
  p.x = static_cast<const uint8_t*>(d->x);
  p.x_is_fp8 = d->x_dtype == TK_E4M3;
  p.x_stride_m = d->x_stride_m;
  p.x_row_scale = d->x_row_scale;
  p.w = static_cast<const uint8_t*>(d->w);
  p.w_scale = static_cast<const uint8_t*>(d->w_mx_scale);
  p.ws_stride_e = d->ws_stride_e;
  p.ws_stride_n = d->ws_stride_n;
  p.w_col_scale = d->w_col_scale;
  p.wcs_stride_e = d->wcs_stride_e;
  p.bias = d->bias;
  p.bias_stride_e = d->bias_stride_e;
  p.bias_is_f32 = d->bias_dtype == TK_F32;
  if (d->bias && d->bias_dtype != TK_F32 && d->bias_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: bias must be fp32 or bf16");
  p.gather = d->gather_indx;
  p.scatter = d->scatter_indx;
  p.scatter_len = d->scatter_len;
  p.gammas = d->gammas;
  p.gammas_is_f32 = d->gammas_dtype == TK_F32;
  if (d->gammas && d->gammas_dtype != TK_F32 && d->gammas_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: gammas must be fp32 or bf16");
  p.slice_sizes = d->slice_sizes;
  p.slice_offs = d->slice_offs;
  p.block_offs = d->block_offs;
  p.block_sched = d->block_schedule;
  p.n_slices = d->n_slices;
  p.M = d->M;
  p.N = d->N;
  p.K = d->K;
  p.y = static_cast<uint16_t*>(d->y);
  p.y_stride_m = d->y_stride_m;
  p.alpha = d->act_alpha;
  p.limit = d->act_limit;
  p.has_limit = d->act_has_limit;
  p.y_vec = (d->y_stride_m % 8 == 0) && ((reinterpret_cast<uintptr_t>(d->y) & 15) == 0);
  p.bias_vec = d->bias && (d->bias_stride_e % 4 == 0) && ((reinterpret_cast<uintptr_t>(d->bias) & 15) == 0);
  p.grid_n = 0;
  p.idle_cus = d->idle_cus;
  p.tile_counters = d->tile_counters;
  p.y_bytes = 0;
  p.combine_k = 0;
  p.combine_out = nullptr;
  p.combine_stride = 0;
  p.combine_counters = nullptr;
  if (d->combine_k > 0) {
    const bool decode_tile = d->block_m == 16 || d->block_m == 32;
    if (!(d->w_layout == TK_W_TILED && d->w_dtype == TK_E2M1 && d->x_dtype == TK_BF16 && !d->x_mx_scale))
      return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the fused top-k combine needs bf16 activations and tiled MXFP4 weights");
    // block_m 16 / 32: arrival counters per (token, fragment); block_m >= 64: the persistent kernel's tile counters
    if (!d->scatter_indx || !d->combine_out || !(decode_tile ? d->combine_counters != nullptr : d->tile_counters != nullptr) || d->activation != TK_ACT_NONE)
      return fail(TK_ERR_INVALID, "tk_moe_gemm: the fused top-k combine needs scatter_indx, combine_out, its counters (combine_counters at block_m 16 / 32, tile_counters above) and no activation");
    if (!decode_tile && (d->N % 8 || d->combine_stride_m % 8 || (reinterpret_cast<uintptr_t>(d->combine_out) & 15)))
      return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the fused top-k combine at block_m >= 64 needs N %% 8 == 0 and 16-byte aligned rows of combine_out");
    if (d->scatter_len % d->combine_k) return fail(TK_ERR_INVALID, "tk_moe_gemm: scatter_len %d is not a multiple of combine_k %d", d->scatter_len, d->combine_k);
    const int64_t yb = (int64_t)d->scatter_len * d->y_stride_m * 2;
    if (yb >= (int64_t)1 << 31 || d->y_stride_m % 4 || (reinterpret_cast<uintptr_t>(d->y) & 7) || d->N % 4)
      return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the fused top-k combine needs N %% 4 == 0 and 8-byte aligned output rows spanning less than 2 GiB");
    p.y_bytes = (uint32_t)yb;
    p.combine_k = d->combine_k;
    p.combine_out = static_cast<uint16_t*>(d->combine_out);
    p.combine_stride = d->combine_stride_m;
    p.combine_counters = d->combine_counters;
  }
  p.betas = d->betas;
  p.betas_is_f32 = d->betas_dtype == TK_F32;
  if (d->betas && d->betas_dtype != TK_F32 && d->betas_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: betas must be fp32 or bf16");
  p.has_out_alpha = d->has_out_alpha != 0;
  p.out_alpha = d->out_alpha;
  p.acc_in = static_cast<const uint16_t*>(d->acc_in);
  p.acc_in_stride_m = d->acc_in_stride_m;
  const bool extras = d->betas || d->has_out_alpha || d->acc_in;
  if (d->acc_in && d->scatter_indx) return fail(TK_ERR_INVALID, "tk_moe_gemm: acc_in is not supported together with scatter_indx");
  if (extras && d->combine_k > 0) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: betas / out_alpha / acc_in are not supported together with the fused top-k combine");
  p.x_mx_scale = static_cast<const uint8_t*>(d->x_mx_scale);
  p.xs_stride_m = d->xs_stride_m;
  p.y_mx_scale = static_cast<uint8_t*>(d->y_mx_scale);
  p.ys_stride_m = d->ys_stride_m;
  p.y_mx_kind = d->y_dtype;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool swiglu = d->activation == TK_ACT_SWIGLU;
  if (d->w_layout == TK_W_TILED && d->w_dtype == TK_E4M3) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with e4m3 weights");
    if (d->block_m != 128 && d->block_m != 256) return fail(TK_ERR_INVALID, "tk_moe_gemm: tiled e4m3 weights take block_m 128 or 256 (got %d)", d->block_m);
    if (d->K < 16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: K must be at least 16 (got %d)", d->K);
    if ((reinterpret_cast<uintptr_t>(d->w) & 15) || d->w_stride_e % 16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: tiled weights must be 16-byte aligned");
    const int64_t nfr = cdiv(d->N, 32), nst = cdiv(d->K, 256);  // stages of 256 = two 4 KiB blocks per fragment
    if (d->n_slices > 1 && d->w_stride_e < nfr * nst * 8192) return fail(TK_ERR_INVALID, "tk_moe_gemm: expert stride smaller than one tiled expert");
    p.w_stride_e = d->w_stride_e;
    p.w_nst = (int32_t)nst;
    if (d->block_m == 256) {
      // 256 x 256 tiles; the kernel addresses activation rows with 32-bit byte offsets from x
      const int64_t x_rows = d->x_rows > 0 ? d->x_rows : (d->gather_indx ? 0 : d->M);
      if (x_rows > 0 && d->x_stride_m >= 0 && x_rows * d->x_stride_m < ((int64_t)1 << 32)) return gemm_launch_f8w(p, d->grid_m, swiglu, st);
    }
    return gemm_launch_f8n(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (mx_act) {
    // MXFP8 activations x tiled MXFP4 weights on the scaled MFMA
    if (d->w_layout != TK_W_TILED || d->w_dtype != TK_E2M1 || !d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MXFP8 activations go with tiled MXFP4 weights");
    if (d->block_m != 128 && d->block_m != 256) return fail(TK_ERR_INVALID, "tk_moe_gemm: MXFP8 activations take block_m 128 or 256 (got %d)", d->block_m);
    if (d->K % 32 || d->K < 128) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MXFP8 activations need K %% 32 == 0 and K >= 128 (got %d)", d->K);
    if (d->x_row_scale || d->w_col_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: per-row / per-column scales are not supported with MXFP8 activations");
    if ((reinterpret_cast<uintptr_t>(d->w) & 15) || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w_mx_scale) & 3) || d->ws_stride_e % 4) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: tiled weights must be 16-byte aligned");
    const int64_t nfr = cdiv(d->N, 32), nst = cdiv(d->K, 128);
    if (d->n_slices > 1 && (d->w_stride_e < nfr * nst * 2048 || d->ws_stride_e < nfr * nst * 128)) return fail(TK_ERR_INVALID, "tk_moe_gemm: expert stride smaller than one tiled expert");
    if (mx_out && extras) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: betas / out_alpha / acc_in are not supported together with an MX-quantised output");
    if (mx_out) {
      const int64_t n_out = swiglu ? d->N / 2 : d->N;
      if (n_out % 32) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: an MX-quantised output needs N_out %% 32 == 0 (got %lld)", (long long)n_out);
      p.y_vec = (d->y_stride_m % 8 == 0) && ((reinterpret_cast<uintptr_t>(d->y) & 7) == 0);
    }
    p.w_stride_e = d->w_stride_e;
    p.w_nst = (int32_t)nst;
    {
      // The persistent form of the kernel (units of work two ahead, branch-free epilogue through buffer resources) needs
      // 32-bit addressable activations and scales, aligned output rows in less than 2 GiB, the ragged metadata in LDS and
      // the plain epilogue; anything else runs the tile-at-a-time form.
      const int64_t x_rows = d->x_rows > 0 ? d->x_rows : (d->gather_indx ? 0 : d->M);
      const int64_t n_out = swiglu ? d->N / 2 : d->N;
      const int64_t y_rows = d->scatter_indx ? d->scatter_len : d->M;
      const int64_t elem = mx_out ? 1 : 2, piece = swiglu ? 4 : 8;
      const int64_t y_bytes = y_rows * d->y_stride_m * elem;
      // (K >= 512: the persistent form reads a row's activation scales sixteen at a time)
      bool fast = d->K >= 512 && x_rows > 0 && x_rows * d->x_stride_m < ((int64_t)1 << 32) && x_rows * d->xs_stride_m < ((int64_t)1 << 32) && d->x_stride_m >= 0 &&
                  d->xs_stride_m >= 0 && !extras && d->n_slices <= kMetaSlices && y_bytes > 0 && y_bytes < ((int64_t)1 << 31) && d->y_stride_m >= 0;
      if (mx_out)
        fast = fast && p.y_vec && y_rows * d->ys_stride_m < ((int64_t)1 << 31) && d->ys_stride_m >= 0;
      else
        fast = fast && p.y_vec && d->y_stride_m >= cdiv(n_out, piece) * piece;
      p.y_bytes = fast ? (uint32_t)y_bytes : 0u;
    }
    return gemm_launch_mx8n(p, d->block_m, d->grid_m, swiglu, mx_out, st);
  }
  if (d->w_layout == TK_W_TILED) {
    if (d->w_dtype != TK_E2M1 || !d->w_mx_scale || d->x_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the tiled weight layout holds MXFP4 weights for bf16 activations");
    if (d->block_m != 16 && d->block_m != 32 && d->block_m != 64 && d->block_m != 128 && d->block_m != 256) return fail(TK_ERR_INVALID, "tk_moe_gemm: block_m must be 16, 32, 64, 128 or 256 (got %d)", d->block_m);
    if (d->block_m >= 64 && extras) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: betas / out_alpha / acc_in need block_m 16 or 32 with tiled MXFP4 weights");
    if (mx_out_bf16 && d->combine_k > 0) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the fused top-k combine needs a bf16 output");
    if (d->block_m >= 64) {
      // the prefill kernels address activation rows with 32-bit byte offsets from x
      if (d->gather_indx && d->x_rows <= 0)
        return fail(TK_ERR_INVALID, "tk_moe_gemm: x_rows is required with gather_indx for tiled MXFP4 weights at block_m >= 64 (the kernel addresses x with 32-bit offsets and must know its extent)");
      const int64_t rows = d->x_rows > 0 ? d->x_rows : d->M;
      if (d->x_stride_m * 2 >= (int64_t)1 << 32 || rows * d->x_stride_m * 2 > (int64_t)1 << 32)
        return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activations of 4 GiB and more are not supported with tiled MXFP4 weights (%lld rows, row stride %lld)", (long long)rows, (long long)d->x_stride_m);
    }
    if (mx_out_bf16) {
      // y_stride_m counts stored elements: bytes, two e2m1 codes each for TK_E2M1.  A lane stores the 4 (swiglu) or 8 values
      // of its column group in one piece of 2 to 8 bytes.
      const int64_t n_out = swiglu ? d->N / 2 : d->N;
      const int64_t y_rows = d->scatter_indx ? d->scatter_len : d->M;
      const int64_t row_bytes = d->y_dtype == TK_E2M1 ? n_out / 2 : n_out;
      const int64_t y_bytes = y_rows * d->y_stride_m;
      if (n_out % 32) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: an MX-quantised output needs N_out %% 32 == 0 (got %lld)", (long long)n_out);
      if (d->y_stride_m % 8 || (reinterpret_cast<uintptr_t>(d->y) & 7) || d->y_stride_m < row_bytes || d->ys_stride_m < n_out / 32)
        return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: rows of an MX-quantised output must be 8-byte aligned and hold the row (row stride %lld for %lld bytes)", (long long)d->y_stride_m, (long long)row_bytes);
      if (y_bytes >= (int64_t)1 << 31 || y_rows * d->ys_stride_m >= (int64_t)1 << 31) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: outputs of 2 GiB and more are not supported with tiled MXFP4 weights");
      p.y_bytes = (uint32_t)y_bytes;
    } else if (d->block_m >= 64) {
      // the prefill kernels store through a buffer resource with 16-byte (8-byte with swiglu) pieces per lane: rows
      // must be 16-byte aligned and long enough to take the last piece whole
      const int64_t n_out = swiglu ? d->N / 2 : d->N;
      const int64_t piece = swiglu ? 4 : 8;
      const int64_t y_rows = d->scatter_indx ? d->scatter_len : d->M;
      const int64_t y_bytes = y_rows * d->y_stride_m * 2;
      if (!p.y_vec || d->y_stride_m < cdiv(n_out, piece) * piece)
        return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: with tiled MXFP4 weights at block_m >= 64 output rows must be 16-byte aligned and padded to a multiple of %lld columns (row stride %lld for %lld columns)", (long long)piece, (long long)d->y_stride_m, (long long)n_out);
      if (y_bytes >= (int64_t)1 << 31) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: outputs of 2 GiB and more are not supported with tiled MXFP4 weights");
      p.y_bytes = (uint32_t)y_bytes;
    }
    if (d->block_m >= 64 && d->n_slices > kMetaSlices) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: at most %d slices with tiled MXFP4 weights at block_m >= 64 (got %d)", kMetaSlices, d->n_slices);
    if (d->block_m >= 64 && (d->x_row_scale || d->w_col_scale)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: per-row / per-column scales are not supported with tiled MXFP4 weights at block_m >= 64");
    if ((reinterpret_cast<uintptr_t>(d->w) & 15) || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w_mx_scale) & 3) || d->ws_stride_e % 4) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: tiled weights must be 16-byte aligned");
    const int64_t nfr = cdiv(d->N, 32), nst = cdiv(d->K, 128);
    if (d->n_slices > 1 && (d->w_stride_e < nfr * nst * 2048 || d->ws_stride_e < nfr * nst * 128)) return fail(TK_ERR_INVALID, "tk_moe_gemm: expert stride smaller than one tiled expert");
    p.w_stride_e = d->w_stride_e;
    p.w_nst = (int32_t)nst;
    if (d->block_m <= 32) return gemm_launch_mxd(p, d->block_m, d->grid_m, swiglu, st);
    if (mx_out_bf16) return gemm_launch_mxn_mx(p, d->block_m, d->grid_m, swiglu, st);
    return gemm_launch_mxn(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_layout != TK_W_STRIDED) return fail(TK_ERR_INVALID, "tk_moe_gemm: bad w_layout %d", d->w_layout);
  if (d->w_stride_k != 1) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weights must be K-contiguous (stride_k == 1)");
  if (d->w_dtype == TK_E2M1) {
    if (!d->w_mx_scale) return fail(TK_ERR_INVALID, "tk_moe_gemm: e2m1 weights need MX scales");
    if (d->ws_stride_k != 1) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales must be K-contiguous");
    if (d->K % 32) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: K must be a multiple of 32 for MX weights (got %d)", d->K);
    if (d->w_stride_n % 16 || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: packed weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e;
    p.w_stride_n = d->w_stride_n;
    return gemm_launch_strided(p, WK_MXFP4, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_BF16) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with bf16 weights");
    if (d->w_stride_n % 8 || d->w_stride_e % 8 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e * 2;
    p.w_stride_n = d->w_stride_n * 2;
    return gemm_launch_strided(p, WK_BF16, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_F16) {
    // fp16 x fp16 -> fp16 (v_mfma_f32_*_f16); same data path as bf16
    if (d->x_dtype != TK_F16 || d->y_dtype != TK_F16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: fp16 weights go with fp16 activations and an fp16 output");
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with fp16 weights");
    if (d->w_stride_n % 8 || d->w_stride_e % 8 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e * 2;
    p.w_stride_n = d->w_stride_n * 2;
    return gemm_launch_strided(p, WK_F16, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_E4M3) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with e4m3 weights");
    if (d->w_stride_n % 16 || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e;
    p.w_stride_n = d->w_stride_n;
    return gemm_launch_strided(p, WK_FP8, d->block_m, d->grid_m, swiglu, st);
  }
  return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight dtype %d is not supported", d->w_dtype);
}

