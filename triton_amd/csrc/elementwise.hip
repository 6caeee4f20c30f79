// Small HBM-bound kernels around the expert GEMMs: standalone swiglu, the k-way combine
// (masked / scaled sum over the expert dimension) and per-row dynamic fp8 quantisation.
#include "mx_math.h"

namespace tk {
namespace {

template <int DT>
__device__ inline float ld(const void* p, int64_t i) {
  if (DT == TK_F32) return static_cast<const float*>(p)[i];
  if (DT == TK_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
}
template <int DT>
__device__ inline void st(void* p, int64_t i, float v) {
  if (DT == TK_F32)
    static_cast<float*>(p)[i] = v;
  else if (DT == TK_BF16)
    static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else
    static_cast<uint16_t*>(p)[i] = f32_to_f16_bits(v);
}

// out[m, j] = s * (l + 1), s = g * sigmoid(alpha * g), (g, l) = (a[m, 2j], a[m, 2j+1]) after clamping.
template <int DT>
__global__ __launch_bounds__(256) void swiglu_kernel(const void* a, int64_t stride_am, void* out, int64_t stride_om,
                                                     int64_t M, int64_t N, float alpha, float limit, int has_limit,
                                                     const int32_t* n_rows_ptr) {
  if (n_rows_ptr) M = *n_rows_ptr < M ? *n_rows_ptr : M;
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / N, j = i - m * N;
    float g = ld<DT>(a, m * stride_am + 2 * j);
    float l = ld<DT>(a, m * stride_am + 2 * j + 1);
    if (has_limit) {
      g = fminf(g, limit);
      l = fminf(fmaxf(l, -limit), limit);
    }
    const float s = g / (1.0f + expf(-alpha * g));
    st<DT>(out, m * stride_om + j, fmaf(s, l, s));
  }
}

// y[a, c] = sum_j mask[a, j, c] ? x[a, j, c] * scale[a, j, c] : 0, fp32 accumulation in j order.
template <int DT>
__global__ __launch_bounds__(256) void reduce_mid_kernel(const void* x, int64_t sx0, int64_t sx1, int64_t A, int64_t K,
                                                         int64_t C, const uint8_t* mask, int64_t sm0, int64_t sm1,
                                                         int64_t sm2, const float* scale, int64_t ss0, int64_t ss1,
                                                         int64_t ss2, void* y, int64_t sy0) {
  const int64_t total = A * C;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t a = i / C, c = i - a * C;
    float acc = 0.f;
    for (int64_t j = 0; j < K; ++j) {
      float v = ld<DT>(x, a * sx0 + j * sx1 + c);
      if (scale) v *= scale[a * ss0 + j * ss1 + c * ss2];
      if (mask && !mask[a * sm0 + j * sm1 + c * sm2]) v = 0.f;
      acc += v;
    }
    st<DT>(y, a * sy0 + c, acc);
  }
}

// Backward of the reduction: dx[a, j, c] = mask[a, j, c] ? dy[a, c] * scale[a, j, c] : 0 (dx contiguous [A, K, C]).
template <int DT>
__global__ __launch_bounds__(256) void reduce_mid_backward_kernel(const void* dy, int64_t sdy0, int64_t A, int64_t K, int64_t C,
                                                                  const uint8_t* mask, int64_t sm0, int64_t sm1, int64_t sm2,
                                                                  const float* scale, int64_t ss0, int64_t ss1, int64_t ss2, void* dx) {
  const int64_t total = A * K * C;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % C, aj = i / C;
    const int64_t j = aj % K, a = aj / K;
    float v = ld<DT>(dy, a * sdy0 + c);
    if (scale) v *= scale[a * ss0 + j * ss1 + c * ss2];
    if (mask && !mask[a * sm0 + j * sm1 + c * sm2]) v = 0.f;
    st<DT>(dx, i, v);
  }
}

// Fast path of the k-way combine: bf16, no mask / scale, 8 columns (16 bytes) per thread, fp32 sum in j order.
__global__ __launch_bounds__(256) void reduce_mid_bf16x8_kernel(const uint16_t* x, int64_t sx0, int64_t sx1, int64_t A, int K,
                                                                int C8, uint16_t* y, int64_t sy0) {
  const int64_t total = A * (int64_t)C8;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t a = i / C8;
    const int c = (int)(i - a * C8) * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const uint16_t* src = x + a * sx0 + c;
    for (int j = 0; j < K; ++j) {
      const uint4 v = *reinterpret_cast<const uint4*>(src + j * sx1);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[2 * q] += bits_f32(w[q] << 16);
        acc[2 * q + 1] += bits_f32(w[q] & 0xFFFF0000u);
      }
    }
    uint32_t o[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = (uint32_t)f32_to_bf16_bits(acc[2 * q]) | ((uint32_t)f32_to_bf16_bits(acc[2 * q + 1]) << 16);
    *reinterpret_cast<uint4*>(y + a * sy0 + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// Per-row dynamic quantisation to OCP e4m3: s = amax / 448 (1 for an all-zero row), q = sat(x / s).
// One wave per row; the row is read twice (second pass hits L2), 16 bytes per lane and load where aligned.
__global__ __launch_bounds__(256) void quant_fp8_rows_kernel(const uint16_t* x, int64_t stride_m, int64_t M, int64_t K,
                                                             uint8_t* q, int64_t stride_qm, float* scales) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const uint16_t* xr = x + row * stride_m;
  uint8_t* qr = q + row * stride_qm;
  // 16-byte loads / 8-byte stores when rows allow it (the scalar loop covers the rest of the row, or all of it)
  const bool vec = ((reinterpret_cast<uintptr_t>(xr) & 15) | (reinterpret_cast<uintptr_t>(qr) & 7)) == 0;
  const int64_t kv = vec ? (K & ~int64_t(7)) : 0;
  float m = 0.f;
#pragma unroll 4
  for (int64_t k = lane * 8; k < kv; k += 512) {  // unrolled so that several 16-byte loads per lane are in flight
    const uint4 v = *reinterpret_cast<const uint4*>(xr + k);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) m = fmaxf(m, fmaxf(fabsf(bits_f32(w[i] << 16)), fabsf(bits_f32(w[i] & 0xFFFF0000u))));
  }
  for (int64_t k = kv + lane; k < K; k += 64) m = fmaxf(m, fabsf(bf16_bits_to_f32(xr[k])));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  float s = m / 448.0f;
  if (s == 0.f) s = 1.0f;
  if (lane == 0) scales[row] = s;
#pragma unroll 4
  for (int64_t k = lane * 8; k < kv; k += 512) {
    const uint4 v = *reinterpret_cast<const uint4*>(xr + k);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    // hardware conversion (OCP e4m3 on this GPU, round to nearest even) of the clamped quotients, two per instruction
    float q8[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q8[2 * i] = mx_clamp(bits_f32(w[i] << 16) / s, 448.0f);
      q8[2 * i + 1] = mx_clamp(bits_f32(w[i] & 0xFFFF0000u) / s, 448.0f);
    }
    int o0 = 0, o1 = 0;
    o0 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[0], q8[1], o0, false);
    o0 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[2], q8[3], o0, true);
    o1 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[4], q8[5], o1, false);
    o1 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[6], q8[7], o1, true);
    *reinterpret_cast<uint2*>(qr + k) = make_uint2((uint32_t)o0, (uint32_t)o1);
  }
  for (int64_t k = kv + lane; k < K; k += 64) qr[k] = (uint8_t)e4m3_byte(mx_clamp(bf16_bits_to_f32(xr[k]) / s, 448.0f));
}

// The same with the row held in registers between the two passes (rows 16-byte aligned, K a multiple of 8 and at most
// NV * 2048): a WORKGROUP per row, NV 16-byte pieces per thread, the row maximum through LDS, one read of x instead of
// two.  (With a wave per row and two passes some thirty rows per CU are between their passes at any time, 29 MB per XCD
// at K = 14336 against an L2 of 4 MB, so the second pass came from memory again: 16384 x 14336 in 189 us, 134 us this
// way.  A wave per row with the row in registers needs 4 NV registers per lane for a row four times as long per lane and
// was slower than two passes from 8192 elements on; for rows of 4096 it took 25 us at 8192 rows, this takes 21.)
template <int NV>
__global__ __launch_bounds__(256) void quant_fp8_rows_wg_kernel(const uint16_t* x, int64_t stride_m, int64_t M, int64_t K, uint8_t* q,
                                                                int64_t stride_qm, float* scales) {
  __shared__ float wmax_s[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * stride_m;
  uint8_t* qr = q + row * stride_qm;
  uint4 v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t k = (int64_t)i * 2048 + tid * 8;
    v[i] = k < K ? *reinterpret_cast<const uint4*>(xr + k) : make_uint4(0u, 0u, 0u, 0u);
  }
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
    for (int c = 0; c < 4; ++c) m = fmaxf(m, fmaxf(fabsf(bits_f32(w[c] << 16)), fabsf(bits_f32(w[c] & 0xFFFF0000u))));
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  if (lane == 0) wmax_s[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(wmax_s[0], wmax_s[1]), fmaxf(wmax_s[2], wmax_s[3]));
  float s = m / 448.0f;
  if (s == 0.f) s = 1.0f;
  if (tid == 0) scales[row] = s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t k = (int64_t)i * 2048 + tid * 8;
    const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    float q8[8];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      q8[2 * c] = mx_clamp(bits_f32(w[c] << 16) / s, 448.0f);
      q8[2 * c + 1] = mx_clamp(bits_f32(w[c] & 0xFFFF0000u) / s, 448.0f);
    }
    int o0 = 0, o1 = 0;
    o0 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[0], q8[1], o0, false);
    o0 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[2], q8[3], o0, true);
    o1 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[4], q8[5], o1, false);
    o1 = __builtin_amdgcn_cvt_pk_fp8_f32(q8[6], q8[7], o1, true);
    if (k < K) *reinterpret_cast<uint2*>(qr + k) = make_uint2((uint32_t)o0, (uint32_t)o1);
  }
}

int grid_for(int64_t total) {
  int64_t g = cdiv(total, 256);
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

// Measurement aid: nothing but MFMA instructions on register operands, eight independent accumulators per wave, one
// or two waves per SIMD.  Its rate under the board's power cap is the ceiling a GEMM of that MFMA class can be compared
// with on this machine (the published peaks assume the 2.4 GHz engine clock, which the cap does not sustain under MFMA
// load).  Operands are lane-dependent, finite and of mixed sign so that the multipliers toggle as they do on real data.
// KIND 0: v_mfma_f32_32x32x16_bf16 (32768 FLOP); 1: v_mfma_f32_32x32x64_f8f6f4 on e4m3 operands (131072 FLOP);
// 2: v_mfma_f32_16x16x32_bf16 (16384 FLOP, sixteen accumulators per wave so that the pipe stays full).
typedef int i32x8_probe_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_probe __attribute__((ext_vector_type(4)));
template <int KIND>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* out, int iters) {
  constexpr bool FP8 = KIND == 1;
  uint32_t raw[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t t = ((uint32_t)threadIdx.x * 8u + e + 37u * i) * 2654435761u;
      // bf16 pairs / e4m3 quads with exponents near 1.0 (no NaN or infinity patterns)
      raw[i][e] = FP8 ? ((t & 0x87878787u) | 0x30303030u) : ((t & 0x807F807Fu) | 0x3F003F00u);
    }
  f32x16_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
  if constexpr (KIND == 2) {
    typedef float f32x4_probe __attribute__((ext_vector_type(4)));
    f32x4_probe acc4[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc4[j] = f32x4_probe{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const u32x4_probe a = {raw[j & 3][0], raw[j & 3][1], raw[j & 3][2], raw[j & 3][3]};
        const u32x4_probe b = {raw[(j >> 2) & 3][4], raw[(j >> 2) & 3][5], raw[(j >> 2) & 3][6], raw[(j >> 2) & 3][7]};
        acc4[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc4[j], 0, 0, 0);
      }
    }
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[j & 7][e] += acc4[j][e];
  } else
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (FP8) {
        const i32x8_probe_t a = {(int)raw[j & 3][0], (int)raw[j & 3][1], (int)raw[j & 3][2], (int)raw[j & 3][3],
                                 (int)raw[j & 3][4], (int)raw[j & 3][5], (int)raw[j & 3][6], (int)raw[j & 3][7]};
        const int bi = (j >> 1) & 3;
        const i32x8_probe_t b = {(int)raw[bi][7], (int)raw[bi][6], (int)raw[bi][5], (int)raw[bi][4],
                                 (int)raw[bi][3], (int)raw[bi][2], (int)raw[bi][1], (int)raw[bi][0]};
        acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
      } else {
        const u32x4_probe a = {raw[j & 3][0], raw[j & 3][1], raw[j & 3][2], raw[j & 3][3]};
        const u32x4_probe b = {raw[(j >> 1) & 3][4], raw[(j >> 1) & 3][5], raw[(j >> 1) & 3][6], raw[(j >> 1) & 3][7]};
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc[j], 0, 0, 0);
      }
    }
  }
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) sum += acc[j][e];
  if (sum == 123456.789f) out[blockIdx.x * 256 + threadIdx.x] = sum;  // keeps the loop; practically never true
}

}  // namespace
}  // namespace tk

using namespace tk;

extern "C" int32_t tk_probe_mfma(float* out, int32_t n_workgroups, int32_t iters, int32_t kind, tk_stream_t stream) {
  if (!out || n_workgroups <= 0 || iters <= 0 || kind < 0 || kind > 2) return fail(TK_ERR_INVALID, "tk_probe_mfma: bad arguments");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (kind == 1)
    hipLaunchKernelGGL(probe_mfma_kernel<1>, dim3((unsigned)n_workgroups), dim3(256), 0, s, out, iters);
  else if (kind == 2)
    hipLaunchKernelGGL(probe_mfma_kernel<2>, dim3((unsigned)n_workgroups), dim3(256), 0, s, out, iters);
  else
    hipLaunchKernelGGL(probe_mfma_kernel<0>, dim3((unsigned)n_workgroups), dim3(256), 0, s, out, iters);
  return check_launch("probe_mfma_kernel");
}

extern "C" int32_t tk_swiglu(const void* a, int32_t dtype, int64_t M, int64_t n_out, int64_t stride_am, void* out,
                             int64_t stride_om, float alpha, float limit, int32_t has_limit, const int32_t* n_rows_ptr,
                             tk_stream_t stream) {
  if (M < 0 || n_out < 0) return fail(TK_ERR_INVALID, "tk_swiglu: negative size");
  if (M == 0 || n_out == 0) return TK_OK;
  if (!a || !out) return fail(TK_ERR_INVALID, "tk_swiglu: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = grid_for(M * n_out);
  if (dtype == TK_BF16)
    hipLaunchKernelGGL(swiglu_kernel<TK_BF16>, dim3(grid), dim3(256), 0, s, a, stride_am, out, stride_om, M, n_out, alpha, limit, has_limit, n_rows_ptr);
  else if (dtype == TK_F16)
    hipLaunchKernelGGL(swiglu_kernel<TK_F16>, dim3(grid), dim3(256), 0, s, a, stride_am, out, stride_om, M, n_out, alpha, limit, has_limit, n_rows_ptr);
  else if (dtype == TK_F32)
    hipLaunchKernelGGL(swiglu_kernel<TK_F32>, dim3(grid), dim3(256), 0, s, a, stride_am, out, stride_om, M, n_out, alpha, limit, has_limit, n_rows_ptr);
  else
    return fail(TK_ERR_UNSUPPORTED, "tk_swiglu: dtype %d", dtype);
  return check_launch("swiglu_kernel");
}

extern "C" int32_t tk_reduce_mid(const void* x, int32_t dtype, int64_t A, int64_t K, int64_t C, int64_t sx0, int64_t sx1,
                                 const void* mask, int64_t sm0, int64_t sm1, int64_t sm2, const float* scale, int64_t ss0,
                                 int64_t ss1, int64_t ss2, void* y, int64_t sy0, tk_stream_t stream) {
  if (A < 0 || K < 0 || C < 0) return fail(TK_ERR_INVALID, "tk_reduce_mid: negative size");
  if (A == 0 || C == 0) return TK_OK;
  if (!x || !y) return fail(TK_ERR_INVALID, "tk_reduce_mid: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t* m = static_cast<const uint8_t*>(mask);
  if (dtype == TK_BF16 && !mask && !scale && C % 8 == 0 && sx0 % 8 == 0 && sx1 % 8 == 0 && sy0 % 8 == 0 && K <= 0x7FFFFFFF && C <= 0x7FFFFFFF &&
      ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0) {
    hipLaunchKernelGGL(reduce_mid_bf16x8_kernel, dim3(grid_for(A * (C / 8))), dim3(256), 0, s, static_cast<const uint16_t*>(x), sx0, sx1, A,
                       (int)K, (int)(C / 8), static_cast<uint16_t*>(y), sy0);
    return check_launch("reduce_mid_bf16x8_kernel");
  }
  const int grid = grid_for(A * C);
  if (dtype == TK_BF16)
    hipLaunchKernelGGL(reduce_mid_kernel<TK_BF16>, dim3(grid), dim3(256), 0, s, x, sx0, sx1, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, y, sy0);
  else if (dtype == TK_F16)
    hipLaunchKernelGGL(reduce_mid_kernel<TK_F16>, dim3(grid), dim3(256), 0, s, x, sx0, sx1, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, y, sy0);
  else if (dtype == TK_F32)
    hipLaunchKernelGGL(reduce_mid_kernel<TK_F32>, dim3(grid), dim3(256), 0, s, x, sx0, sx1, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, y, sy0);
  else
    return fail(TK_ERR_UNSUPPORTED, "tk_reduce_mid: dtype %d", dtype);
  return check_launch("reduce_mid_kernel");
}

extern "C" int32_t tk_reduce_mid_backward(const void* dy, int32_t dtype, int64_t A, int64_t K, int64_t C, int64_t sdy0, const void* mask,
                                          int64_t sm0, int64_t sm1, int64_t sm2, const float* scale, int64_t ss0, int64_t ss1,
                                          int64_t ss2, void* dx, tk_stream_t stream) {
  if (A < 0 || K < 0 || C < 0) return fail(TK_ERR_INVALID, "tk_reduce_mid_backward: negative size");
  if (A == 0 || K == 0 || C == 0) return TK_OK;
  if (!dy || !dx) return fail(TK_ERR_INVALID, "tk_reduce_mid_backward: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t* m = static_cast<const uint8_t*>(mask);
  const int grid = grid_for(A * K * C);
  if (dtype == TK_BF16)
    hipLaunchKernelGGL(reduce_mid_backward_kernel<TK_BF16>, dim3(grid), dim3(256), 0, s, dy, sdy0, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, dx);
  else if (dtype == TK_F16)
    hipLaunchKernelGGL(reduce_mid_backward_kernel<TK_F16>, dim3(grid), dim3(256), 0, s, dy, sdy0, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, dx);
  else if (dtype == TK_F32)
    hipLaunchKernelGGL(reduce_mid_backward_kernel<TK_F32>, dim3(grid), dim3(256), 0, s, dy, sdy0, A, K, C, m, sm0, sm1, sm2, scale, ss0, ss1, ss2, dx);
  else
    return fail(TK_ERR_UNSUPPORTED, "tk_reduce_mid_backward: dtype %d", dtype);
  return check_launch("reduce_mid_backward_kernel");
}

extern "C" int32_t tk_quant_fp8_rows(const void* x, int32_t dtype, int64_t M, int64_t K, int64_t stride_m, void* q,
                                     int64_t stride_qm, float* scales, tk_stream_t stream) {
  if (M < 0 || K < 0) return fail(TK_ERR_INVALID, "tk_quant_fp8_rows: negative size");
  if (M == 0) return TK_OK;
  if (!x || !q || !scales) return fail(TK_ERR_INVALID, "tk_quant_fp8_rows: null pointer");
  if (dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_quant_fp8_rows: input must be bf16");
  const dim3 grid((unsigned)cdiv(M, 4)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  uint8_t* qd = static_cast<uint8_t*>(q);
  const bool aligned = K % 8 == 0 && stride_m % 8 == 0 && stride_qm % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0;
  if (aligned && K > 2048 && K <= 32768 && M <= 0x7FFFFFFF) {
    const dim3 rows((unsigned)M);
    if (K <= 4096)
      hipLaunchKernelGGL(quant_fp8_rows_wg_kernel<2>, rows, block, 0, st, xs, stride_m, M, K, qd, stride_qm, scales);
    else if (K <= 16384)
      hipLaunchKernelGGL(quant_fp8_rows_wg_kernel<8>, rows, block, 0, st, xs, stride_m, M, K, qd, stride_qm, scales);
    else
      hipLaunchKernelGGL(quant_fp8_rows_wg_kernel<16>, rows, block, 0, st, xs, stride_m, M, K, qd, stride_qm, scales);
    return check_launch("quant_fp8_rows_wg_kernel");
  }
  hipLaunchKernelGGL(quant_fp8_rows_kernel, grid, block, 0, st, xs, stride_m, M, K, qd, stride_qm, scales);
  return check_launch("quant_fp8_rows_kernel");
}
