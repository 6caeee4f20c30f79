// Pieces shared by the expert-GEMM kernels of this library (one translation unit per kernel family, so that they
// compile side by side): the kernel parameter block, the tile claimer of the persistent kernels, MFMA fragment
// traits, the shared epilogue and the launch helpers.  `tk_moe_gemm` (moe_gemm.hip) validates a descriptor, fills a
// GemmParams and calls one family's `gemm_launch_*`.
#pragma once
#include <atomic>
#include <mutex>
#include <type_traits>
#include <unordered_map>

#include "common.h"
#include "mx_math.h"

namespace tk {

enum { WK_BF16 = 0, WK_MXFP4 = 1, WK_FP8 = 2, WK_F16 = 3 };  // weight storage: bf16, packed e2m1 + e8m0 scales, e4m3, fp16 (with fp16 activations)

struct GemmParams {
  const uint8_t* x;    // bf16 or e4m3 rows
  int32_t x_is_fp8;
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
  int32_t y_vec;     // output rows allow 16-byte vector stores
  int32_t bias_vec;  // bias rows allow 16-byte vector loads
  int32_t w_nst;     // tile-native weight layout: K-stages of 128 per column fragment
  int32_t total_tiles;  // persistent kernels, non-ragged case: row blocks x column tiles
  int32_t idle_cus;     // persistent kernels: compute units to leave without a workgroup
  int32_t* tile_counters;  // persistent kernels: 32 zeroed words (tile claiming: 0..8; prefill combine: 9..31), or null
  uint32_t y_bytes;        // persistent MXFP4 kernels: bytes of the output buffer that rows may be written to (< 2 GiB)
  int32_t combine_k;          // decode kernel: > 0 = sum the k rows of every token into combine_out (fused top-k combine)
  uint16_t* combine_out;      // bf16 [tokens, N]
  int64_t combine_stride;
  int32_t* combine_counters;  // zeroed [tokens * ceil(N / 32)] words, left zero
  const uint8_t* x_mx_scale;  // e8m0 block scales of MXFP8 activations [rows, K/32], or null
  int64_t xs_stride_m;
  uint8_t* y_mx_scale;        // e8m0 block scales of an MX-quantised output [rows, N_out/32], or null
  int64_t ys_stride_m;
  int32_t y_mx_kind;          // TK_E4M3, TK_E5M2 or TK_E2M1: the element type of an MX-quantised output
  // options of the shared epilogue only (the host keeps them away from the kernels with an epilogue of their own)
  const void* betas;          // per expert-sorted row multiplier of the bias, or null
  int32_t betas_is_f32;
  int32_t has_out_alpha;      // acc *= out_alpha behind the bias, in front of the activation
  float out_alpha;
  const uint16_t* acc_in;     // tensor of the output's shape and type added to the result (behind the gate weight), or null
  int64_t acc_in_stride_m;
};

// one entry per kernel family; each returns a TK_* status
int32_t gemm_launch_strided(const GemmParams& p, int wk, int block_m, int grid_m, bool swiglu, hipStream_t st);
int32_t gemm_launch_mxn(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st);
int32_t gemm_launch_mxn_mx(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st);  // block_m 128 / 256, MX-quantised output
int32_t gemm_launch_mxd(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st);
int32_t gemm_launch_f8n(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st);
int32_t gemm_launch_f8w(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st);  // 256 x 256 tiles (row blocks of 256)
int32_t gemm_launch_mx8n(const GemmParams& p, int block_m, int grid_m, bool swiglu, bool mx_out, hipStream_t st);

// Slices (experts) whose row and block offsets the persistent MXFP4 prefill kernel keeps in LDS: a tile's coordinates
// then cost LDS reads instead of a chain of dependent global loads.  The host refuses more slices than this.
constexpr int kMetaSlices = 1024;

namespace {

template <int I>
using template_int = std::integral_constant<int, I>;

// f(integral_constant<int, I>) for I in [B, E), fully expanded at compile time
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
// byte offset that a buffer resource drops (stores) or reads as zero (loads): buffers span less than 2 GiB (host check)
constexpr uint32_t kDroppedStore = 0x80000000u;
typedef int32_t i32x8_t __attribute__((ext_vector_type(8)));



// Persistent kernels hand out tiles either statically (round r gives workgroup b tile r * grid + remap(b)) or, when the
// caller supplies `tile_counters`, dynamically: the tile list is cut into 8 contiguous queues, one per XCD, and a
// workgroup claims the next tile of its XCD's queue with an atomic increment (tiles that share weights or
// activations keep running next to each other under one L2); when its queue is empty it takes from the other
// queues in ring order.  Tiles cost different amounts (4 or 5 row fragments, partly filled column tiles), so a
// static deal waits for the slowest tile of every round.  The claim for the NEXT tile is issued when a tile starts and
// read when it ends, so the atomic's latency is hidden behind the tile's K loop.  Words 0..7 = next index of each
// queue, word 8 = workgroups that have finished; the last one to finish clears all nine words, so the counters
// are zero again when the kernel ends (launches that share the words must not overlap in time).

struct TileClaimer {
  int32_t* ctr;
  int live;
  int myq;
  int pending;   // thread 0: index returned by the claim in flight
  __device__ __forceinline__ int qbeg(int q) const { return (int)(((int64_t)live * q) >> 3); }
  // Workgroups that start on queue q number ((grid - q + 7) / 8); each takes two tiles of the queue without asking
  // (indices blockIdx.x / 8 and that plus their number), so the counters count from twice their number.
  __device__ __forceinline__ int qwgs(int q) const { return ((int)gridDim.x - q + 7) >> 3; }
  __device__ __forceinline__ int qfirst(int q) const { return 2 * qwgs(q); }
  // second tile of this workgroup (thread-uniform, no memory access), -1 if its queue is shorter than that
  __device__ __forceinline__ int second() const {
    const int t = qbeg(myq) + (int)(blockIdx.x >> 3) + qwgs(myq);
    return t < qbeg(myq + 1) ? t : -1;
  }
  // first tile of this workgroup (thread-uniform, no memory access), -1 if its queue is shorter than that
  __device__ __forceinline__ int init(int32_t* c, int live_tiles) {
    ctr = c;
    live = live_tiles;
    myq = blockIdx.x & 7;
    pending = 0;
    const int t = qbeg(myq) + (int)(blockIdx.x >> 3);
    return t < qbeg(myq + 1) ? t : -1;
  }
  // thread 0: start the claim of this workgroup's next tile (own queue)
  // (the result goes through a variable that is undefined in the other lanes: merging it with the previous value
  // would make every lane wait for the atomic to return right here)
  __device__ __forceinline__ void issue() {
    int fresh;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wsometimes-uninitialized"
    if (threadIdx.x == 0) fresh = atomicAdd(&ctr[myq], 1);
    pending = fresh;
#pragma clang diagnostic pop
  }
  // thread 0: tile id of the claim in flight, or of another queue when the own one is exhausted; -1 = no tile left.
  // The other queues' counters are read together first, so a workgroup that finds everything taken pays two
  // memory round trips, not eight.
  __device__ __forceinline__ int resolve() {
    int t = qbeg(myq) + qfirst(myq) + pending;
    if (t < qbeg(myq + 1)) return t;
    int seen[8];
#pragma unroll
    for (int i = 1; i < 8; ++i) seen[i] = __hip_atomic_load(&ctr[(myq + i) & 7], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int i = 1; i < 8; ++i) {
      const int q = (myq + i) & 7;
      if (qbeg(q) + qfirst(q) + seen[i] >= qbeg(q + 1)) continue;  // counters only grow: taken stays taken
      t = qbeg(q) + qfirst(q) + atomicAdd(&ctr[q], 1);
      if (t < qbeg(q + 1)) return t;
    }
    return -1;
  }
  // thread 0, once, after the workgroup's last claim: count it as finished; the last workgroup clears the counters
  __device__ __forceinline__ void finish() {
    if (threadIdx.x == 0) {
      __threadfence();
      if (atomicAdd(&ctr[8], 1) == (int)gridDim.x - 1) {
        __threadfence();
        for (int i = 0; i < 9; ++i) atomicExch(&ctr[i], 0);
      }
    }
  }
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

// s * (linear + 1), s = gate * sigmoid(alpha * gate).  `nalpha_log2e` = -alpha * log2(e); `limit` = +inf when the
// activation has no limit.  v_med3_f32 clamps in one instruction; exp2 and the reciprocal are the hardware
// approximations (1 ulp each).
__device__ __forceinline__ float swiglu_f(float gate, float lin, float nalpha_log2e, float limit) {
  gate = __builtin_amdgcn_fmed3f(gate, -INFINITY, limit);
  lin = __builtin_amdgcn_fmed3f(lin, -limit, limit);
  const float s = gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(nalpha_log2e * gate));
  return fmaf(s, lin, s);
}

// two fp32 -> packed bf16 pair (round to nearest even), low half = a
__device__ inline uint32_t pack_bf16x2(float a, float b) {
  f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// output conversions of the shared epilogue: bf16, or fp16 for the fp16 x fp16 kernel
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
template <bool F16>
__device__ __forceinline__ uint32_t pack_out2(float a, float b) {
  if constexpr (F16) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  } else {
    return pack_bf16x2(a, b);
  }
}
template <bool F16>
__device__ __forceinline__ uint16_t cvt_out(float a) {
  if constexpr (F16)
    return f32_to_f16_bits(a);
  else
    return f32_to_bf16_bits(a);
}

// FM = 16: v_mfma_f32_16x16x32_bf16 (lane = row % 16, 4 k-groups of 32 per 128-wide sub-stage).
// FM = 32: v_mfma_f32_32x32x16_bf16 (lane = row % 32, 2 k-groups of 64), the full-rate shape on gfx950.
template <int FM>
struct Frag;
template <>
struct Frag<16> {
  typedef f32x4_t acc_t;
  static constexpr int NACC = 4;
  static __device__ __forceinline__ acc_t mma(bf16x8_t a, bf16x8_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // the same registers read as eight fp16 values
  static __device__ __forceinline__ acc_t mma_f16(bf16x8_t a, bf16x8_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  // accumulator register i of lane group h holds fragment row (= output column) n_of(i, h)
  static __device__ __forceinline__ int n_of(int i, int h) { return h * 4 + i; }
};
template <>
struct Frag<32> {
  typedef f32x16_t acc_t;
  static constexpr int NACC = 16;
  static __device__ __forceinline__ acc_t mma(bf16x8_t a, bf16x8_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ acc_t mma_f16(bf16x8_t a, bf16x8_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ int n_of(int i, int h) { return (i >> 2) * 8 + h * 4 + (i & 3); }
};

// Epilogue shared by the GEMM kernels.  acc[f][j] is the FM x FM fragment of column fragment f (first column
// ncol0 + f*FM) and row fragment j (tile rows (j*WM + mw)*FM ..); register i of a lane in lane group h holds
// output column Frag::n_of(i, h) of row lr.  Order: row/column scales, bias, activation, gate weight,
// (scattered) store.  Everything the rows and columns need from memory is fetched before the first store.
template <int FM, int WM, int MFW, int NFW, bool SWIGLU, bool F16OUT = false>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, typename Frag<FM>::acc_t (&acc)[NFW][MFW], int expert,
                                              int off_m, int start_m, int eM, int ncol0, bool full_n, int mw, int lr, int h) {
  typedef Frag<FM> FR;
  const int N = p.N;
  const int NOUT = SWIGLU ? N / 2 : N;
  // per-row items; rows past the slice read the slice's last row (no divergent branches around the loads)
  float gam[MFW], rsc[MFW];
  int64_t dst[MFW];
  bool ok[MFW];
  int srow[MFW];
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const int row = off_m + (j * WM + mw) * FM + lr;  // row inside the slice
    ok[j] = row < eM;
    srow[j] = start_m + (ok[j] ? row : eM - 1);       // row in expert-sorted order
    gam[j] = 1.0f;
    rsc[j] = 1.0f;
    dst[j] = srow[j];
  }
  if (p.gammas) {
#pragma unroll
    for (int j = 0; j < MFW; ++j) gam[j] = load_scalar(p.gammas, srow[j], p.gammas_is_f32);
  }
  if (p.scatter) {
#pragma unroll
    for (int j = 0; j < MFW; ++j) {
      const int sr = srow[j] < p.scatter_len ? srow[j] : p.scatter_len - 1;
      const int v = p.scatter[sr];
      dst[j] = srow[j] < p.scatter_len ? v : -1;
    }
  }
  if (p.x_row_scale) {
    int src[MFW];
#pragma unroll
    for (int j = 0; j < MFW; ++j) src[j] = p.gather ? p.gather[srow[j]] : srow[j];
#pragma unroll
    for (int j = 0; j < MFW; ++j) rsc[j] = p.x_row_scale[src[j]];
  }
#pragma unroll
  for (int j = 0; j < MFW; ++j) ok[j] = ok[j] && dst[j] >= 0;
  if (p.x_row_scale || p.w_col_scale) {  // fp8-style per-row x per-column scales
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) {
        const int n = ncol0 + f * FM + FR::n_of(i, h);
        float cs = 1.0f;
        if (p.w_col_scale && n < N) cs = p.w_col_scale[expert * p.wcs_stride_e + n];
#pragma unroll
        for (int j = 0; j < MFW; ++j) acc[f][j][i] *= rsc[j] * cs;
      }
  }
  float beta[MFW];
#pragma unroll
  for (int j = 0; j < MFW; ++j) beta[j] = 1.0f;
  if (p.betas) {
#pragma unroll
    for (int j = 0; j < MFW; ++j) beta[j] = load_scalar(p.betas, srow[j], p.betas_is_f32);
  }
  if (p.bias) {
    float b4[NFW][FR::NACC / 4][4];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int q = 0; q < FR::NACC / 4; ++q) {
        const int n0 = ncol0 + f * FM + FR::n_of(4 * q, h);  // 4 consecutive columns
        const int64_t bo = expert * p.bias_stride_e + n0;
        if (full_n && p.bias_vec) {
          if (p.bias_is_f32) {
            const float4 t = *reinterpret_cast<const float4*>(static_cast<const float*>(p.bias) + bo);
            b4[f][q][0] = t.x, b4[f][q][1] = t.y, b4[f][q][2] = t.z, b4[f][q][3] = t.w;
          } else {
            const uint2 t = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p.bias) + bo);
            b4[f][q][0] = bits_f32(t.x << 16), b4[f][q][1] = bits_f32(t.x & 0xFFFF0000u);
            b4[f][q][2] = bits_f32(t.y << 16), b4[f][q][3] = bits_f32(t.y & 0xFFFF0000u);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) b4[f][q][i] = n0 + i < N ? load_scalar(p.bias, bo + i, p.bias_is_f32) : 0.f;
        }
      }
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int q = 0; q < FR::NACC / 4; ++q)
#pragma unroll
        for (int j = 0; j < MFW; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[f][j][4 * q + i] = p.betas ? fmaf(b4[f][q][i], beta[j], acc[f][j][4 * q + i]) : acc[f][j][4 * q + i] + b4[f][q][i];
  }
  if (p.has_out_alpha) {
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int j = 0; j < MFW; ++j)
#pragma unroll
        for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] *= p.out_alpha;
  }
  // VW consecutive output columns per lane: 4 as the MFMA leaves them (16x16), or 8 after the two lane
  // halves of a 32x32 fragment exchange their 4-column groups (v_permlane32_swap)
  constexpr int VW = FM == 32 ? 8 : 4;
  constexpr int NU = FR::NACC / VW;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  const bool fast = full_n && p.y_vec;  // every column of the tile exists and rows take vector stores
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    float v[NFW][NU][VW];
    int n0[NFW][NU];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        if constexpr (FM == 32) {
          // registers 8u..8u+3 hold columns 16u + 4h + i, registers 8u+4..8u+7 columns 16u + 8 + 4h + i
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            uint32_t lo = f32_bits(acc[f][j][8 * u + i]), hi = f32_bits(acc[f][j][8 * u + 4 + i]);
            auto r = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);  // lo's upper half <-> hi's lower half
            v[f][u][i] = bits_f32(r[0]);
            v[f][u][4 + i] = bits_f32(r[1]);
          }
          n0[f][u] = ncol0 + f * FM + 16 * u + 8 * h;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[f][u][i] = acc[f][j][4 * u + i];
          n0[f][u] = ncol0 + f * FM + FR::n_of(4 * u, h);
        }
      }
    if (!ok[j]) continue;  // one divergent region per row fragment
    uint16_t* yrow = p.y + dst[j] * p.y_stride_m;
    const float g = gam[j];
    if (p.acc_in) {
      // out = act(...) * gate + acc_in[row, column]: fold the gate weight in here and add, element by element (an
      // option off the tuned paths)
      const uint16_t* arow = p.acc_in + dst[j] * p.acc_in_stride_m;
#pragma unroll
      for (int f = 0; f < NFW; ++f)
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          if (SWIGLU) {
            const int o0 = n0[f][u] / 2;
#pragma unroll
            for (int i = 0; i < VW / 2; ++i) {
              if (o0 + i < NOUT) {
                const float a = F16OUT ? f16_bits_to_f32(arow[o0 + i]) : bf16_bits_to_f32(arow[o0 + i]);
                yrow[o0 + i] = cvt_out<F16OUT>(swiglu_f(v[f][u][2 * i], v[f][u][2 * i + 1], nalpha_log2e, limit) * g + a);
              }
            }
          } else {
#pragma unroll
            for (int i = 0; i < VW; ++i) {
              if (n0[f][u] + i < N) {
                const float a = F16OUT ? f16_bits_to_f32(arow[n0[f][u] + i]) : bf16_bits_to_f32(arow[n0[f][u] + i]);
                yrow[n0[f][u] + i] = cvt_out<F16OUT>(v[f][u][i] * g + a);
              }
            }
          }
        }
      continue;
    }
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        if (SWIGLU) {
          float r[VW / 2];
#pragma unroll
          for (int i = 0; i < VW / 2; ++i) r[i] = swiglu_f(v[f][u][2 * i], v[f][u][2 * i + 1], nalpha_log2e, limit) * g;
          const int o0 = n0[f][u] / 2;
          if (fast) {
            uint32_t w[VW / 4];
#pragma unroll
            for (int i = 0; i < VW / 4; ++i) w[i] = pack_out2<F16OUT>(r[2 * i], r[2 * i + 1]);
            if constexpr (VW == 8)
              *reinterpret_cast<uint2*>(yrow + o0) = make_uint2(w[0], w[VW / 4 - 1]);
            else
              *reinterpret_cast<uint32_t*>(yrow + o0) = w[0];
          } else {
#pragma unroll
            for (int i = 0; i < VW / 2; ++i)
              if (o0 + i < NOUT) yrow[o0 + i] = cvt_out<F16OUT>(r[i]);
          }
        } else {
          if (fast) {
            uint32_t w[VW / 2];
#pragma unroll
            for (int i = 0; i < VW / 2; ++i) w[i] = pack_out2<F16OUT>(v[f][u][2 * i] * g, v[f][u][2 * i + 1] * g);
            if constexpr (VW == 8)
              *reinterpret_cast<uint4*>(yrow + n0[f][u]) = make_uint4(w[0], w[1], w[VW / 2 - 2], w[VW / 2 - 1]);
            else
              *reinterpret_cast<uint2*>(yrow + n0[f][u]) = make_uint2(w[0], w[1]);
          } else {
#pragma unroll
            for (int i = 0; i < VW; ++i)
              if (n0[f][u] + i < N) yrow[n0[f][u] + i] = cvt_out<F16OUT>(v[f][u][i] * g);
          }
        }
      }
  }
}

// Raises a kernel's dynamic LDS limit above 64 KiB, once per (kernel, device): the table is keyed on the kernel's
// address, so every template instantiation (the swiglu and the plain variant of one tile shape included) has an
// entry of its own; bit d of an entry = done on device d.
inline int32_t allow_dynamic_lds(const void* kern, int bytes) {
  if (bytes <= 64 * 1024) return TK_OK;
  static std::mutex mu;
  static std::unordered_map<const void*, uint64_t> done;
  int dev = 0;
  const bool known = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64;
  if (known) {
    std::lock_guard<std::mutex> lock(mu);
    auto it = done.find(kern);
    if (it != done.end() && (it->second >> dev & 1ull)) return TK_OK;
  }
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(TK_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", bytes, hipGetErrorString(e));
  if (known) {
    std::lock_guard<std::mutex> lock(mu);
    done[kern] |= 1ull << dev;
  }
  return TK_OK;
}

// compute units of the current device (cached per device id; racing first calls store the same value)
inline int device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// compute units a persistent grid may fill when `idle` of them are to stay free (at least one is used)
inline int busy_cu_count(int idle) {
  const int n = device_cu_count() - (idle > 0 ? idle : 0);
  return n > 0 ? n : 1;
}

}  // namespace

// Epilogue of the persistent prefill kernels.  Everything a tile's rows and columns need (bias as fp32, gate weight,
// destination row or -1) was fetched ahead and sits in LDS: bias_s[BN] by tile column, gam_s / dst_s [BM] by tile
// row.  Order: bias, activation, gate weight, (scattered) store.  The bias is added as each accumulator register
// is read for the last time (a pass of its own over the accumulators would move all of them between the
// accumulation and the vector registers twice more).
// Every lane executes every store instruction: rows without a destination and columns past N get a byte offset
// beyond the buffer resource's range, which the hardware drops.  With no branch around a store the number of
// stores between two loads is the same on every path, so the compiler's vmcnt waits for loads issued BEFORE the
// epilogue (the next unit's first operands) do not wait for these stores to drain.

// NFV = leading column fragments of the wave that hold real columns; the others skip the arithmetic and issue their
// stores with the dropped offset, so that the number of stores is the same on every path.
// HOIST: all LDS operands (a lane's 16 * NFW bias values, its rows' gate weights and destinations) are read into
// registers up front, one LDS round trip instead of one per row fragment and column group; for kernels whose registers
// are free behind the K loop.
template <int G, int MFW, int NFW, int NFV, bool SWIGLU, bool HOIST = false>
__device__ __forceinline__ void staged_epilogue(const GemmParams& p, f32x16_t (&acc)[NFW][MFW], __amdgpu_buffer_rsrc_t yrsrc, const float* bias_s,
                                                const float* gam_s, const int* dst_s, int ncol_tile, int ncol0, int grp, int lr, int h) {
  const int NOUT = SWIGLU ? p.N / 2 : p.N;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  const uint32_t row_bytes = (uint32_t)(p.y_stride_m * 2);
  f32x4_t bh[NFW][2][2];
  float gh[MFW];
  int dh[MFW];
  if constexpr (HOIST) {
#pragma unroll
    for (int f = 0; f < NFV; ++f)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        bh[f][u][0] = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 4 * h);
        bh[f][u][1] = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 8 + 4 * h);
      }
#pragma unroll
    for (int j = 0; j < MFW; ++j) {
      gh[j] = gam_s[(j * G + grp) * 32 + lr];
      dh[j] = dst_s[(j * G + grp) * 32 + lr];
    }
  }
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const int r = (j * G + grp) * 32 + lr;
    const float g = HOIST ? gh[j] : gam_s[r];
    const int dst = HOIST ? dh[j] : dst_s[r];
    const uint32_t row_off = dst >= 0 ? (uint32_t)dst * row_bytes : kDroppedStore;
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (f >= NFV) {
          if (SWIGLU)
            __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{0u, 0u}, yrsrc, kDroppedStore, 0, 0);
          else
            __builtin_amdgcn_raw_buffer_store_b128(u32x4_t{0u, 0u, 0u, 0u}, yrsrc, kDroppedStore, 0, 0);
          continue;
        }
        // registers 8u..8u+3 hold columns 16u + 4h + i, registers 8u+4..8u+7 columns 16u + 8 + 4h + i: after the two
        // lane halves exchange their 4-column groups a lane holds 8 consecutive columns from 16u + 8h
        float v[8];
        // bias of the two column groups (zeros without a bias), re-read from LDS for every row fragment: keeping all
        // of a lane's 32 bias values in registers costs more than the reads
        const f32x4_t b0 = HOIST ? bh[f][u][0] : *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 4 * h);
        const f32x4_t b1 = HOIST ? bh[f][u][1] : *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 8 + 4 * h);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t lo = f32_bits(acc[f][j][8 * u + i] + b0[i]), hi = f32_bits(acc[f][j][8 * u + 4 + i] + b1[i]);
          auto sw = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);
          v[i] = bits_f32(sw[0]);
          v[4 + i] = bits_f32(sw[1]);
        }
        const int n0 = ncol0 + f * 32 + 16 * u + 8 * h;  // first of this lane's 8 columns
        if (SWIGLU) {
          float o[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = swiglu_f(v[2 * i], v[2 * i + 1], nalpha_log2e, limit) * g;
          const int o0 = n0 / 2;
          const uint32_t off = (o0 < NOUT && dst >= 0) ? row_off + (uint32_t)o0 * 2u : kDroppedStore;
          const u32x2_t w = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
          __builtin_amdgcn_raw_buffer_store_b64(w, yrsrc, off, 0, 0);
        } else {
          const uint32_t off = (n0 < NOUT && dst >= 0) ? row_off + (uint32_t)n0 * 2u : kDroppedStore;
          u32x4_t w;
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(v[2 * i] * g, v[2 * i + 1] * g);
          __builtin_amdgcn_raw_buffer_store_b128(w, yrsrc, off, 0, 0);
        }
      }
  }
}


// MX-quantised output of the persistent prefill kernels (matmul_details/_matmul.py:593-637): blocks of 32 output columns of the
// fp32 accumulator (after bias, activation and gate weight), one e8m0 scale byte per block (round-up rule) to y_mx_scale, values
// as e4m3, e5m2 or packed e2m1 (p.y_mx_kind) to y.  The operands of rows and columns are taken
// from LDS (bias_s by tile column, gam_s / dst_s by tile row, fetched a unit ahead) and with no branch around a store:
// rows without a destination, columns past the end and the lanes that do not write a block's scale byte store to an
// offset beyond the range of their buffer resource, which the hardware drops.
template <int MFW, int NFW, bool SWIGLU>
__device__ __forceinline__ void staged_mx_epilogue(const GemmParams& p, f32x16_t (&acc)[NFW][MFW], __amdgpu_buffer_rsrc_t yrsrc,
                                                   __amdgpu_buffer_rsrc_t ysrsrc, const float* bias_s, const float* gam_s, const int* dst_s,
                                                   int ncol_tile, int ncol0, int lr, int h) {
  const int NOUT = SWIGLU ? p.N / 2 : p.N;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  constexpr int VO = SWIGLU ? 4 : 8;
  constexpr int NB = SWIGLU ? 1 : NFW;
  // every LDS operand up front: one round trip for the unit
  f32x4_t bh[NFW][2][2];
  float gh[MFW];
  int dh[MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      bh[f][u][0] = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 4 * h);
      bh[f][u][1] = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 8 + 4 * h);
    }
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    gh[j] = gam_s[j * 32 + lr];
    dh[j] = dst_s[j * 32 + lr];
  }
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const float g = gh[j];
    const int dst = dh[j];
    float o[NFW][2][VO];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          auto sw = __builtin_amdgcn_permlane32_swap(f32_bits(acc[f][j][8 * u + i] + bh[f][u][0][i]), f32_bits(acc[f][j][8 * u + 4 + i] + bh[f][u][1][i]), false, false);
          v[i] = bits_f32(sw[0]);
          v[4 + i] = bits_f32(sw[1]);
        }
#pragma unroll
        for (int i = 0; i < VO; ++i) o[f][u][i] = SWIGLU ? swiglu_f(v[2 * i], v[2 * i + 1], nalpha_log2e, limit) * g : v[i] * g;
      }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      // block maximum of |o|: fmaxf returns its other operand for a NaN, so a NaN never wins and the block's scale comes
      // from its finite values.  (N_out is a multiple of 32: a block lies below it whole or not at all, and one that does
      // not is not stored.)
      float m = 0.f;
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < VO; ++i) m = __builtin_fmaxf(m, __builtin_fabsf(o[f][u][i]));
      }
      {
        // the other lane half's maximum: after the swap the first register holds both halves' lanes 0..31, the second both
        // halves' lanes 32..63
        auto sw = __builtin_amdgcn_permlane32_swap(f32_bits(m), f32_bits(m), false, false);
        m = __builtin_fmaxf(bits_f32(sw[0]), bits_f32(sw[1]));
      }
      const int kind = p.y_mx_kind;  // uniform
      const uint32_t sbits = mx_scale_bits(m, kind, TK_MX_ROUND_UP);
      const float inv = mx_inv_scale(sbits);
      const int blk_col0 = SWIGLU ? ncol0 / 2 : ncol0 + b * 32;
      const uint32_t soff = (dst >= 0 && h == 0 && blk_col0 < NOUT) ? (uint32_t)dst * (uint32_t)p.ys_stride_m + (uint32_t)(blk_col0 >> 5) : kDroppedStore;
      __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(sbits >> 23), ysrsrc, soff, 0, 0);
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int col0 = SWIGLU ? (ncol0 + f * 32 + 16 * u + 8 * h) / 2 : ncol0 + f * 32 + 16 * u + 8 * h;
          // No clamp in front of the conversion: the scale is the smallest power of two >= max / max_q (the rounded quotient
          // of an fp32 by 448 = 1.75 * 2^8, 57344 = 1.75 * 2^15 or 6 = 1.5 * 2^2 is a power of two only when the exact one
          // is), scaling by a power of two is exact, so |o * inv| <= max_q for every finite block; with an infinite maximum
          // inv is 0.  The three kinds issue the same number of stores (the wait counts of loads issued ahead stay exact).
          float qv[VO];
#pragma unroll
          for (int i = 0; i < VO; ++i) qv[i] = o[f][u][i] * inv;
          const bool live = dst >= 0 && col0 < NOUT;
          if (kind == TK_E2M1) {
            // two codes per byte, even column in the low nibble; NaN saturates like the infinity of its sign (mxfp.py:298-327)
#pragma unroll
            for (int i = 0; i < VO; ++i) qv[i] = qv[i] != qv[i] ? __builtin_copysignf(INFINITY, qv[i]) : qv[i];
            uint32_t w = 0;
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, qv[0], qv[1], 1.0f, 0);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, qv[2], qv[3], 1.0f, 1);
            const uint32_t off = live ? (uint32_t)dst * (uint32_t)p.y_stride_m + (uint32_t)(col0 >> 1) : kDroppedStore;
            if constexpr (VO == 8) {
              w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, qv[4], qv[5], 1.0f, 2);
              w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, qv[6], qv[7], 1.0f, 3);
              __builtin_amdgcn_raw_buffer_store_b32(w, yrsrc, off, 0, 0);
            } else {
              __builtin_amdgcn_raw_buffer_store_b16((uint16_t)w, yrsrc, off, 0, 0);
            }
          } else {
            const uint32_t off = live ? (uint32_t)dst * (uint32_t)p.y_stride_m + (uint32_t)col0 : kDroppedStore;
            int w0 = 0, w1 = 0;
            if (kind == TK_E4M3) {
              w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], w0, false);
              w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], w0, true);
              if constexpr (VO == 8) {
                w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], w1, false);
                w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], w1, true);
              }
            } else {
              w0 = __builtin_amdgcn_cvt_pk_bf8_f32(qv[0], qv[1], w0, false);
              w0 = __builtin_amdgcn_cvt_pk_bf8_f32(qv[2], qv[3], w0, true);
              if constexpr (VO == 8) {
                w1 = __builtin_amdgcn_cvt_pk_bf8_f32(qv[4], qv[5], w1, false);
                w1 = __builtin_amdgcn_cvt_pk_bf8_f32(qv[6], qv[7], w1, true);
              }
            }
            if constexpr (VO == 8)
              __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{(uint32_t)w0, (uint32_t)w1}, yrsrc, off, 0, 0);
            else
              __builtin_amdgcn_raw_buffer_store_b32((uint32_t)w0, yrsrc, off, 0, 0);
          }
        }
      }
    }
  }
}


// Top-k combine behind the scatter of a persistent prefill kernel (reduce.py:1143-1165 after matmul_details/_matmul.py:535-569 in the reference,
// a launch of its own there): out[t, :] = sum over j of y[t * k + j, :], fp32 in j order, bf16 result.  The k rows of a
// token come from k experts, i.e. from tiles of workgroups all over the chip, so the sum runs when EVERY workgroup
// has written its tiles: the grid is persistent and fits the GPU (one workgroup per CU).
//   1. a workgroup whose stores have all reached its XCD's L2 counts itself in (per XCD and in total);
//   2. when all have, ONE workgroup per XCD (the first to claim it) has that L2 write its dirty lines back (a release
//      fence; one per L2, not one per wave: every fence walks the whole cache) and reports it;
//   3. when every XCD in use has reported, the rows of y are in memory: the workgroups sum the tokens blockIdx.x,
//      blockIdx.x + grid, ..., reading y around their own L2 (sc0 sc1: lines another XCD wrote are not coherent in it);
//   4. the last workgroup to leave clears the words for the next launch.
// Words of `tile_counters`: 9 arrivals, 10 departures, 11 error (raised, and kept, if a bounded wait runs out),
// 12 XCDs in use, 13 XCDs written back, 16..23 arrivals per XCD, 24..31 write-back claimed per XCD.
template <int NT>
__device__ __forceinline__ void fused_prefill_combine(const GemmParams& p, int tid, int grid) {
  const int N = p.N;
  int32_t* ctr = p.tile_counters;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    xcc &= 7;
    auto wait_for = [&](int32_t* word, int want) {
      int spins = 0;
      while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
        __builtin_amdgcn_s_sleep(16);
        if (++spins > (1 << 22)) {
          atomicOr(&ctr[11], 1);
          break;
        }
      }
    };
    if (__hip_atomic_fetch_add(&ctr[16 + xcc], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
      __hip_atomic_fetch_add(&ctr[12], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_fetch_add(&ctr[9], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    wait_for(&ctr[9], grid);
    if (__hip_atomic_fetch_add(&ctr[24 + xcc], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // this XCD's L2 writes back its dirty lines
      __hip_atomic_fetch_add(&ctr[13], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    wait_for(&ctr[13], __hip_atomic_load(&ctr[12], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  }
  __syncthreads();
  const int k = p.combine_k, T = p.scatter_len / k;
  const int n8 = N >> 3;  // (N is a multiple of 8: host check)
  const __amdgpu_buffer_rsrc_t ysrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);
  const uint32_t row_bytes = (uint32_t)(p.y_stride_m * 2);
  constexpr int kAround = 1 | 16;  // sc0 | sc1
  // The tokens of this workgroup and their 8-column groups form one index space, H items of it per lane and pass:
  // their rows are all requested before any is summed (4 * H 16-byte loads in flight per lane when k <= 4).
  constexpr int H = 2;
  const int n_tok = blockIdx.x < T ? (T - 1 - blockIdx.x) / grid + 1 : 0;
  const int items = n_tok * n8;
  for (int i0 = tid; i0 < items; i0 += H * NT) {
    int tt[H], cc[H];
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const int i = i0 + h * NT;
      const int lt = i / n8;
      tt[h] = i < items ? blockIdx.x + lt * grid : -1;
      cc[h] = i - lt * n8;
    }
    float sum[H][8];
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[h][e] = 0.f;
    for (int j0 = 0; j0 < k; j0 += 4) {
      u32x4_t v[H][4];
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t off =
              (tt[h] >= 0 && j0 + q < k) ? (uint32_t)(tt[h] * k + j0 + q) * row_bytes + (uint32_t)cc[h] * 16u : kDroppedStore;
          v[h][q] = __builtin_amdgcn_raw_buffer_load_b128(ysrc, off, 0, kAround);  // (dropped offsets read zero)
        }
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            sum[h][2 * e] += bits_f32(v[h][q][e] << 16);
            sum[h][2 * e + 1] += bits_f32(v[h][q][e] & 0xFFFF0000u);
          }
    }
#pragma unroll
    for (int h = 0; h < H; ++h)
      if (tt[h] >= 0)
        *reinterpret_cast<u32x4_t*>(p.combine_out + (int64_t)tt[h] * p.combine_stride + cc[h] * 8) =
            u32x4_t{pack_bf16x2(sum[h][0], sum[h][1]), pack_bf16x2(sum[h][2], sum[h][3]), pack_bf16x2(sum[h][4], sum[h][5]),
                    pack_bf16x2(sum[h][6], sum[h][7])};
  }
  __syncthreads();
  if (tid == 0) {
    if (__hip_atomic_fetch_add(&ctr[10], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == grid - 1) {
      for (int w = 9; w < 32; ++w)
        if (w != 11) __hip_atomic_store(&ctr[w], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace tk
