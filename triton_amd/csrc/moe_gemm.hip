// Ragged (grouped) expert GEMM for gfx950 with fused gather, MX dequantisation, bias, swiglu, gate
// scaling and scatter.
//
//   Y[dst(r), :] = act( (X[src(r), :] @ W[e(r)]) * sx[src(r)] * sw[e(r), :] + bias[e(r), :] ) * gamma[r]
//
// Mapping onto CDNA4:
//   * one workgroup = WAVES wave64s computes a tile of BM = 16*MF rows (of ONE expert) by
//     BN = WAVES*NF*16 output columns; each wave owns NF 16-column fragments and ALL rows;
//   * the MFMA is issued "transposed": the A operand is a 16(n) x 32(k) fragment of W^T and the B
//     operand a 32(k) x 16(m) fragment of X^T, so a lane's 4 accumulator registers are 4 CONSECUTIVE
//     output columns of one row (swiglu's (gate, linear) column pairs are lane-local);
//   * weights are K-contiguous per output column ([E, N, K] in memory), which is exactly the MFMA
//     operand order: each lane streams its own column straight from global memory into registers,
//     16 bytes (= 32 e2m1 values = one MX block = one e8m0 scale) per 128-wide K step, and
//     dequantises with v_cvt_scalef32_pk_bf16_fp4; W never passes through LDS and is never
//     dequantised twice;
//   * the (gathered) activation rows are staged once per K step through LDS (double buffered,
//     rows padded by 16 B so that ds_read_b128 of 16 rows is bank-conflict free) and shared by all
//     waves.
#include "common.h"

namespace tk {
namespace {

enum { WK_BF16 = 0, WK_MXFP4 = 1 };

struct GemmParams {
  const uint16_t* x;
  int64_t x_stride_m;
  const float* x_row_scale;
  const uint8_t* w;
  int64_t w_stride_e;  // bytes
  int64_t w_stride_n;  // bytes
  const uint8_t* w_scale;
  int64_t ws_stride_e;
  int64_t ws_stride_n;
  const float* w_col_scale;
  int64_t wcs_stride_e;
  const void* bias;
  int64_t bias_stride_e;
  int32_t bias_is_f32;
  const int32_t* gather;
  const int32_t* scatter;
  int32_t scatter_len;
  const void* gammas;
  int32_t gammas_is_f32;
  const int32_t* slice_sizes;
  const int32_t* slice_offs;
  const int32_t* block_offs;
  const int32_t* block_sched;
  int32_t n_slices;
  int32_t M, N, K;
  uint16_t* y;
  int64_t y_stride_m;
  int32_t grid_n;
  float alpha, limit;
  int32_t has_limit;
  int32_t y_vec;  // output rows allow 8-byte vector stores
};

__device__ inline int xcd_remap(int pid, int total) {
  // Workgroups are dealt round-robin to the 8 XCDs (each with a private L2); renumber so that
  // consecutive tile ids run on the same XCD.
  const int per = total / 8, extra = total % 8;
  const int grp = pid % 8, local = pid / 8;
  return grp * per + (grp < extra ? grp : extra) + local;
}

__device__ inline float load_scalar(const void* p, int64_t i, int is_f32) {
  return is_f32 ? static_cast<const float*>(p)[i] : bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
}

// 8 e2m1 values (one dword, even element in the low nibble) -> 8 bf16 scaled by `scale`.
__device__ inline bf16x8_t dequant8(uint32_t raw, float scale) {
  bf16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(raw, scale, 0);
  bf16x2_t b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(raw, scale, 1);
  bf16x2_t c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(raw, scale, 2);
  bf16x2_t d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(raw, scale, 3);
  bf16x8_t r = {a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
  return r;
}

__device__ inline float swiglu_f(float gate, float lin, float alpha, float limit, int has_limit) {
  if (has_limit) {
    gate = fminf(gate, limit);
    lin = fminf(fmaxf(lin, -limit), limit);
  }
  const float s = gate / (1.0f + __expf(-alpha * gate));
  return fmaf(s, lin, s);
}

template <int WK, int MF, int NF, int WAVES, int KS, bool SWIGLU>
__global__ __launch_bounds__(WAVES * 64) void moe_gemm_kernel(const GemmParams p) {
  constexpr int BM = MF * 16;
  constexpr int BN = WAVES * NF * 16;
  constexpr int NT = WAVES * 64;
  constexpr int KC = 128 * KS;           // K elements per pipeline stage
  constexpr int PITCH = KC * 2 + 16;     // LDS row pitch in bytes
  constexpr int NCHUNK = BM * (KC / 8);  // 16-byte pieces of one X stage
  constexpr int CH = (NCHUNK + NT - 1) / NT;
  constexpr int WREGS = (WK == WK_MXFP4) ? 4 : 16;  // dwords of W per lane per fragment per 128 k

  __shared__ __attribute__((aligned(16))) uint8_t lds[2][BM * PITCH];

  const int pid = xcd_remap(blockIdx.x, gridDim.x);
  const int pid_n = pid % p.grid_n;
  const int pid_m = pid / p.grid_n;
  int expert, off_m, start_m, eM;
  if (p.slice_sizes) {
    if (pid_m >= p.block_offs[p.n_slices]) return;
    const int sched = p.block_sched[pid_m];
    expert = sched & 0xFFFF;
    off_m = (sched >> 16) * BM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    expert = 0;
    off_m = pid_m * BM;
    start_m = 0;
    eM = p.M;
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, g = lane >> 4;
  const int K = p.K, N = p.N;

  // ---- activation staging: this thread's 16-byte pieces ------------------------------------
  const uint16_t* xptr[CH];
  int xk[CH];      // k offset of the piece inside a stage
  int xlds[CH];    // byte offset of the piece inside an LDS stage
  bool xok[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int id = tid + NT * j;
    xok[j] = id < NCHUNK;
    const int r = id / (KC / 8), c = id % (KC / 8);
    int row = off_m + r;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m + c * 8;
    xk[j] = c * 8;
    xlds[j] = r * PITCH + c * 16;
  }
  // ---- weight streaming: this lane's columns -------------------------------------------------
  const int n_base = pid_n * BN + wave * (NF * 16);
  const uint8_t* wptr[NF];
  const uint8_t* sptr[NF];
  bool nok[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int n = n_base + f * 16 + l16;
    nok[f] = n < N;
    const int nn = nok[f] ? n : 0;
    if (WK == WK_MXFP4) {
      wptr[f] = p.w + expert * p.w_stride_e + nn * p.w_stride_n + g * 16;
      sptr[f] = p.w_scale + expert * p.ws_stride_e + nn * p.ws_stride_n + g;
    } else {
      wptr[f] = p.w + expert * p.w_stride_e + nn * p.w_stride_n + g * 64;
      sptr[f] = nullptr;
    }
  }

  f32x4_t acc[NF][MF];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int m = 0; m < MF; ++m) acc[f][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  uint4 xreg[CH];
  uint32_t wreg[2][KS][NF][WREGS];
  uint32_t sreg[2][KS][NF];

  auto load_x = [&](int kc) {
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      if (xok[j] && kc + xk[j] < K)
        xreg[j] = *reinterpret_cast<const uint4*>(xptr[j] + kc);
      else
        xreg[j] = make_uint4(0, 0, 0, 0);
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int j = 0; j < CH; ++j)
      if (xok[j]) *reinterpret_cast<uint4*>(&lds[buf][xlds[j]]) = xreg[j];
  };
  auto load_w = [&](int slot, int kc) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k0 = kc + s * 128 + g * 32;  // first k this lane holds in the sub-step
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        if constexpr (WK == WK_MXFP4) {
          if (nok[f] && k0 < K) {
            const uint4 v = *reinterpret_cast<const uint4*>(wptr[f] + (kc + s * 128) / 2);
            wreg[slot][s][f][0] = v.x;
            wreg[slot][s][f][1] = v.y;
            wreg[slot][s][f][2] = v.z;
            wreg[slot][s][f][3] = v.w;
            sreg[slot][s][f] = sptr[f][(kc + s * 128) / 32];
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) wreg[slot][s][f][i] = 0;
            sreg[slot][s][f] = 127;
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (nok[f] && k0 + 8 * i < K) {
              const uint4 v = *reinterpret_cast<const uint4*>(wptr[f] + (kc + s * 128) * 2 + i * 16);
              wreg[slot][s][f][4 * i + 0] = v.x;
              wreg[slot][s][f][4 * i + 1] = v.y;
              wreg[slot][s][f][4 * i + 2] = v.z;
              wreg[slot][s][f][4 * i + 3] = v.w;
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) wreg[slot][s][f][4 * i + q] = 0;
            }
          }
        }
      }
    }
  };
  auto compute = [&](int buf, int slot) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      float scl[NF];
      if constexpr (WK == WK_MXFP4) {
#pragma unroll
        for (int f = 0; f < NF; ++f) scl[f] = bits_f32(sreg[slot][s][f] << 23);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bf16x8_t xf[MF];
#pragma unroll
        for (int m = 0; m < MF; ++m)
          xf[m] = *reinterpret_cast<const bf16x8_t*>(&lds[buf][(m * 16 + l16) * PITCH + (s * 128 + g * 32 + i * 8) * 2]);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          bf16x8_t wf;
          if constexpr (WK == WK_MXFP4) {
            wf = dequant8(wreg[slot][s][f][i], scl[f]);
          } else {
            uint4 raw = make_uint4(wreg[slot][s][f][4 * i + 0], wreg[slot][s][f][4 * i + 1],
                                   wreg[slot][s][f][4 * i + 2], wreg[slot][s][f][4 * i + 3]);
            wf = __builtin_bit_cast(bf16x8_t, raw);
          }
#pragma unroll
          for (int m = 0; m < MF; ++m) acc[f][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[m], acc[f][m], 0, 0, 0);
        }
      }
    }
  };

  const int nstages = (K + KC - 1) / KC;
  load_x(0);
  load_w(0, 0);
  store_x(0);
  __syncthreads();
  for (int c = 0; c < nstages; ++c) {
    const int cur = c & 1;
    const bool more = c + 1 < nstages;
    if (more) {
      load_x((c + 1) * KC);
      load_w(cur ^ 1, (c + 1) * KC);
    }
    compute(cur, cur);
    if (more) store_x(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue ------------------------------------------------------------------------------
  const int NOUT = SWIGLU ? N / 2 : N;
#pragma unroll
  for (int m = 0; m < MF; ++m) {
    const int row = off_m + m * 16 + l16;  // row inside the slice
    if (row >= eM) continue;
    const int srow = start_m + row;  // row in expert-sorted order
    float rs = 1.0f;
    if (p.x_row_scale) rs = p.x_row_scale[p.gather ? p.gather[srow] : srow];
    float gam = 1.0f;
    if (p.gammas) gam = load_scalar(p.gammas, srow, p.gammas_is_f32);
    int64_t dst = srow;
    if (p.scatter) {
      dst = srow < p.scatter_len ? p.scatter[srow] : -1;
      if (dst < 0) continue;
    }
    uint16_t* yrow = p.y + dst * p.y_stride_m;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int n0 = n_base + f * 16 + g * 4;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + i;
        float a = acc[f][m][i];
        if (n < N) {
          if (p.w_col_scale) a *= rs * p.w_col_scale[expert * p.wcs_stride_e + n];
          else a *= rs;
          if (p.bias) a += load_scalar(p.bias, expert * p.bias_stride_e + n, p.bias_is_f32);
        }
        v[i] = a;
      }
      if (SWIGLU) {
        const int o0 = n0 / 2;
        const float r0 = swiglu_f(v[0], v[1], p.alpha, p.limit, p.has_limit) * gam;
        const float r1 = swiglu_f(v[2], v[3], p.alpha, p.limit, p.has_limit) * gam;
        if (o0 + 1 < NOUT && p.y_vec) {
          *reinterpret_cast<uint32_t*>(yrow + o0) = (uint32_t)f32_to_bf16_bits(r0) | ((uint32_t)f32_to_bf16_bits(r1) << 16);
        } else {
          if (o0 < NOUT) yrow[o0] = f32_to_bf16_bits(r0);
          if (o0 + 1 < NOUT) yrow[o0 + 1] = f32_to_bf16_bits(r1);
        }
      } else {
        if (n0 + 3 < N && p.y_vec) {
          const uint32_t lo = (uint32_t)f32_to_bf16_bits(v[0] * gam) | ((uint32_t)f32_to_bf16_bits(v[1] * gam) << 16);
          const uint32_t hi = (uint32_t)f32_to_bf16_bits(v[2] * gam) | ((uint32_t)f32_to_bf16_bits(v[3] * gam) << 16);
          *reinterpret_cast<uint2*>(yrow + n0) = make_uint2(lo, hi);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n0 + i < N) yrow[n0 + i] = f32_to_bf16_bits(v[i] * gam);
        }
      }
    }
  }
}

template <int WK, int MF, int NF, int WAVES, int KS>
int32_t launch_cfg(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int BN = WAVES * NF * 16;
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, BN);
  const int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  if (swiglu)
    hipLaunchKernelGGL((moe_gemm_kernel<WK, MF, NF, WAVES, KS, true>), dim3((unsigned)grid), dim3(WAVES * 64), 0, st, q);
  else
    hipLaunchKernelGGL((moe_gemm_kernel<WK, MF, NF, WAVES, KS, false>), dim3((unsigned)grid), dim3(WAVES * 64), 0, st, q);
  return check_launch("moe_gemm_kernel");
}

template <int WK>
int32_t launch_wk(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  switch (block_m) {
    case 16:
      return launch_cfg<WK, 1, 2, 4, 2>(p, grid_m, swiglu, st);
    case 32:
      return launch_cfg<WK, 2, 2, 4, 2>(p, grid_m, swiglu, st);
    case 64:
      return launch_cfg<WK, 4, 4, 4, 1>(p, grid_m, swiglu, st);
    case 128:
      return launch_cfg<WK, 8, 4, 4, 1>(p, grid_m, swiglu, st);
    default:
      return fail(TK_ERR_INVALID, "tk_moe_gemm: block_m must be 16, 32, 64 or 128 (got %d)", block_m);
  }
}

}  // namespace
}  // namespace tk

using namespace tk;

extern "C" int32_t tk_moe_gemm(const tk_gemm_desc* d, tk_stream_t stream) {
  if (!d) return fail(TK_ERR_INVALID, "tk_moe_gemm: null descriptor");
  if (d->M < 0 || d->N < 0 || d->K < 0) return fail(TK_ERR_INVALID, "tk_moe_gemm: negative size");
  if (d->M == 0 || d->N == 0 || d->grid_m == 0) return TK_OK;
  if (!d->x || !d->w || !d->y) return fail(TK_ERR_INVALID, "tk_moe_gemm: null operand");
  if (d->x_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activations must be bf16 (dtype %d)", d->x_dtype);
  if (d->y_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: output must be bf16 (dtype %d)", d->y_dtype);
  if (d->w_stride_k != 1) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weights must be K-contiguous (stride_k == 1)");
  if (d->activation != TK_ACT_NONE && d->activation != TK_ACT_SWIGLU) return fail(TK_ERR_INVALID, "tk_moe_gemm: bad activation %d", d->activation);
  if (d->activation == TK_ACT_SWIGLU && d->N % 2) return fail(TK_ERR_INVALID, "tk_moe_gemm: swiglu needs an even N");
  if (d->K % 8) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: K must be a multiple of 8 (got %d)", d->K);
  if (d->x_stride_m % 8 || (reinterpret_cast<uintptr_t>(d->x) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activation rows must be 16-byte aligned");
  if (d->slice_sizes && (!d->slice_offs || !d->block_offs || !d->block_schedule)) return fail(TK_ERR_INVALID, "tk_moe_gemm: incomplete ragged metadata");
  if (d->n_slices >= 65536) return fail(TK_ERR_INVALID, "tk_moe_gemm: at most 65535 slices");
  GemmParams p;
  p.x = static_cast<const uint16_t*>(d->x);
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
  p.y_vec = (d->y_stride_m % 4 == 0) && ((reinterpret_cast<uintptr_t>(d->y) & 7) == 0);
  p.grid_n = 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool swiglu = d->activation == TK_ACT_SWIGLU;
  if (d->w_dtype == TK_E2M1) {
    if (!d->w_mx_scale) return fail(TK_ERR_INVALID, "tk_moe_gemm: e2m1 weights need MX scales");
    if (d->ws_stride_k != 1) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales must be K-contiguous");
    if (d->K % 32) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: K must be a multiple of 32 for MX weights (got %d)", d->K);
    if (d->w_stride_n % 16 || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: packed weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e;
    p.w_stride_n = d->w_stride_n;
    return launch_wk<WK_MXFP4>(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_BF16) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with bf16 weights");
    if (d->w_stride_n % 8 || d->w_stride_e % 8 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e * 2;
    p.w_stride_n = d->w_stride_n * 2;
    return launch_wk<WK_BF16>(p, d->block_m, d->grid_m, swiglu, st);
  }
  return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight dtype %d not supported with bf16 activations", d->w_dtype);
}
