// Ragged (grouped) expert GEMM for gfx950 with fused gather, MX dequantisation, bias, swiglu, gate
// scaling and scatter.
//
//   Y[dst(r), :] = act( (X[src(r), :] @ W[e(r)]) * sx[src(r)] * sw[e(r), :] + bias[e(r), :] ) * gamma[r]
//
// Mapping onto CDNA4:
//   * one workgroup (WM x WN wave64s) computes BM = WM*MFW*FM rows of ONE expert by BN = WN*NFW*FM
//     output columns (FM = 16 or 32, the MFMA fragment edge); the K loop runs in stages of KC = 128*KS;
//   * the MFMA is issued "transposed": the A operand is a 16(n) x 32(k) fragment of W^T and the B
//     operand a 32(k) x 16(m) fragment of X^T, so a lane's 4 accumulator registers are 4 CONSECUTIVE
//     output columns of one row (swiglu's (gate, linear) column pairs are lane-local) and both
//     operands want K-contiguous data, which is how activations ([rows, K]) and the reference's MX
//     weights ([E, N, K/2] in memory) are stored;
//   * both operands are staged through LDS, double buffered, with global loads issued one stage ahead
//     into registers.  Loads are shaped for the texture-address unit: 16 consecutive lanes fetch 256
//     contiguous bytes of one activation row, 4 consecutive lanes the 64 bytes one weight column
//     contributes to a stage; LDS rows are padded by 16 B so the ds_read_b128 of 16 rows / columns is
//     bank-conflict free.  MXFP4 stays packed in LDS (4 bits per weight) together with its e8m0 scales
//     and is expanded in registers by v_cvt_scalef32_pk_bf16_fp4 right before the MFMA;
//   * the rows of a tile are dealt to the WM row-waves in interleaved 16-row fragments and fragments
//     past the expert's last row are skipped, so a nearly empty row block costs almost no MFMA time.
#include <atomic>
#include <mutex>
#include <type_traits>
#include <unordered_map>

#include "common.h"
#include "mx_math.h"

namespace tk {
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
  int32_t* tile_counters;  // persistent kernels: 16 zeroed words for dynamic tile claiming (9 are used), or null
  uint32_t y_bytes;        // persistent MXFP4 kernels: bytes of the output buffer that rows may be written to (< 2 GiB)
  int32_t combine_k;          // decode kernel: > 0 = sum the k rows of every token into combine_out (fused top-k combine)
  uint16_t* combine_out;      // bf16 [tokens, N]
  int64_t combine_stride;
  int32_t* combine_counters;  // zeroed [tokens * ceil(N / 32)] words, left zero
  const uint8_t* x_mx_scale;  // e8m0 block scales of MXFP8 activations [rows, K/32], or null
  int64_t xs_stride_m;
  uint8_t* y_mx_scale;        // e8m0 block scales of an MXFP8 output [rows, N_out/32], or null
  int64_t ys_stride_m;
};

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
          for (int i = 0; i < 4; ++i) acc[f][j][4 * q + i] += b4[f][q][i];
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

template <int WK, int FM, int WM, int WN, int MFW, int NFW, int KS, bool SWIGLU>
__global__ __launch_bounds__(WM * WN * 64) void moe_gemm_kernel(const GemmParams p) {
  typedef Frag<FM> FR;
  constexpr int NT = WM * WN * 64;
  constexpr int BM = WM * MFW * FM;
  constexpr int BN = WN * NFW * FM;
  constexpr int KC = 128 * KS;  // K elements per pipeline stage
  constexpr int NG = 64 / FM;   // k-groups of lanes
  constexpr int KG = 128 / NG;  // k per group per 128-wide sub-stage
  constexpr int SPS = KG / 8;   // MFMA steps per sub-stage
  constexpr bool MX = WK == WK_MXFP4;
  constexpr bool F8 = WK == WK_FP8;  // e4m3 weights AND e4m3 activations, both expanded to bf16 for the MFMA
  constexpr int XE = F8 ? 16 : 8;    // activation elements per 16-byte global piece
  constexpr int XPITCH = KC * 2 + 16;                    // bytes per activation row in LDS
  constexpr int WROW = MX ? KC / 2 : (F8 ? KC : KC * 2);  // weight bytes per column per stage
  constexpr int WPITCH = WROW + 16;                      // MX: the pad holds the KC/32 scale bytes
  constexpr int XBYTES = BM * XPITCH;
  constexpr int STAGE = XBYTES + BN * WPITCH;
  constexpr int XPIECES = BM * (KC / XE);                // 16-byte global pieces per stage
  constexpr int WPIECES = BN * (WROW / 16);
  constexpr int XCH = (XPIECES + NT - 1) / NT;
  constexpr int WCH = (WPIECES + NT - 1) / NT;
  constexpr int SCH = MX ? (BN * KS + NT - 1) / NT : 1;  // scale dwords (4 blocks = 128 k each)
  constexpr bool XFULL = XPIECES % NT == 0, WFULL = WPIECES % NT == 0, SFULL = (BN * KS) % NT == 0;
  static_assert(2 * STAGE <= 160 * 1024, "LDS budget");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  int expert, off_m, start_m, eM, pid_n;
  if (p.slice_sizes) {
    // The grid is an upper bound; renumber only the live tiles so that every XCD gets an equal share.
    const int live = p.block_offs[p.n_slices] * p.grid_n;
    if ((int)blockIdx.x >= live) return;
    const int pid = xcd_remap(blockIdx.x, live);
    // Tiles are ordered (expert, column tile, row block): the row blocks of one expert that share a column
    // tile get consecutive ids, run at the same time on one XCD and stream the same weights through its L2.
    expert = p.block_sched[pid / p.grid_n] & 0xFFFF;
    const int first = p.block_offs[expert];
    const int nb = p.block_offs[expert + 1] - first;
    const int local = pid - first * p.grid_n;
    pid_n = local / nb;
    off_m = (local - pid_n * nb) * BM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    const int pid = xcd_remap(blockIdx.x, gridDim.x);
    pid_n = pid % p.grid_n;
    expert = 0;
    off_m = (pid / p.grid_n) * BM;
    start_m = 0;
    eM = p.M;
  }
  const int rows = (eM - off_m) < BM ? (eM - off_m) : BM;  // valid rows of this tile (>= 1)
  const int nfrag_m = (rows + FM - 1) / FM;                // row fragments that hold valid rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mw = wave % WM, nw = wave / WM;
  const int lr = lane % FM, h = lane / FM;
  const int K = p.K, N = p.N;
  // fragment j of this wave covers tile rows (j*WM + mw)*FM .. +FM; fragments past the last valid row are skipped
  int jcount = 0;
#pragma unroll
  for (int j = 0; j < MFW; ++j) jcount += ((j * WM + mw) < nfrag_m) ? 1 : 0;

  // ---- global -> register staging: this thread's 16-byte pieces -----------------------------
  const uint8_t* xptr[XCH];
  int xk[XCH], xlds[XCH];
  bool xok[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    const int id = tid + NT * j;
    const int r = (id / (KC / XE)) % BM, c = id % (KC / XE);
    xok[j] = (XFULL || id < XPIECES) && r < nfrag_m * FM;  // fragments without valid rows are never read
    int row = off_m + r;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + (src * p.x_stride_m + c * XE) * (F8 ? 1 : 2);
    xk[j] = c * XE;
    xlds[j] = r * XPITCH + c * XE * 2;
  }
  const uint8_t* wptr[WCH];
  int wk[WCH], wlds[WCH];
  bool wok[WCH];
  const int n_tile = pid_n * BN;
#pragma unroll
  for (int j = 0; j < WCH; ++j) {
    const int id = tid + NT * j;
    wok[j] = WFULL || id < WPIECES;
    const int col = (id / (WROW / 16)) % BN, part = id % (WROW / 16);
    int n = n_tile + col;
    n = n < N ? n : N - 1;  // columns past N are computed from a valid column and dropped in the epilogue
    wptr[j] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)n * p.w_stride_n + part * 16;
    wk[j] = MX ? part * 32 : (F8 ? part * 16 : part * 8);
    wlds[j] = XBYTES + col * WPITCH + part * 16;
  }
  const uint8_t* sptr[SCH];
  int sk[SCH], slds[SCH];
  bool sok[SCH];
  if constexpr (MX) {
#pragma unroll
    for (int j = 0; j < SCH; ++j) {
      const int id = tid + NT * j;
      sok[j] = SFULL || id < BN * KS;
      const int col = (id / KS) % BN, part = id % KS;
      int n = n_tile + col;
      n = n < N ? n : N - 1;
      sptr[j] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)n * p.ws_stride_n + part * 4;
      sk[j] = part * 128;
      slds[j] = XBYTES + col * WPITCH + WROW + part * 4;
    }
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  uint4 xreg[XCH];
  uint4 wreg[WCH];
  uint32_t sreg[SCH];

  // TAIL = the stage may reach past K: pieces beyond K are zero-filled (zero weights x finite activations)
  auto load_stage = [&](auto tail_c, int kc) __attribute__((always_inline)) {
    constexpr bool TAIL = decltype(tail_c)::value;
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      if (xok[j] && (!TAIL || kc + xk[j] < K))
        xreg[j] = *reinterpret_cast<const uint4*>(xptr[j] + kc * (F8 ? 1 : 2));
      else
        xreg[j] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < WCH; ++j) {
      if ((WFULL || wok[j]) && (!TAIL || kc + wk[j] < K))
        wreg[j] = *reinterpret_cast<const uint4*>(wptr[j] + (MX ? kc / 2 : (F8 ? kc : kc * 2)));
      else
        wreg[j] = make_uint4(0, 0, 0, 0);
    }
    if constexpr (MX) {
#pragma unroll
      for (int j = 0; j < SCH; ++j) {
        if (!(SFULL || sok[j])) {
          sreg[j] = 0x7F7F7F7Fu;
        } else if (!TAIL) {
          uint32_t v;
          __builtin_memcpy(&v, sptr[j] + kc / 32, 4);  // 4 consecutive e8m0 bytes, any alignment
          sreg[j] = v;
        } else {
          uint32_t v = 0;
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int k0 = kc + sk[j] + 32 * b;
            const uint32_t byte = k0 < K ? (uint32_t)sptr[j][kc / 32 + b] : 127u;
            v |= byte << (8 * b);
          }
          sreg[j] = v;
        }
      }
    }
  };
  auto store_stage = [&](int buf) __attribute__((always_inline)) {
    uint8_t* base = lds + buf * STAGE;
#pragma unroll
    for (int j = 0; j < XCH; ++j)
      if (xok[j]) {
        if constexpr (F8) {  // 16 e4m3 -> 16 bf16 (exact)
          const uint32_t w4[4] = {xreg[j].x, xreg[j].y, xreg[j].z, xreg[j].w};
          uint32_t o[8];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            o[2 * q] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w4[q], 1.0f, false));
            o[2 * q + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w4[q], 1.0f, true));
          }
          *reinterpret_cast<uint4*>(base + xlds[j]) = make_uint4(o[0], o[1], o[2], o[3]);
          *reinterpret_cast<uint4*>(base + xlds[j] + 16) = make_uint4(o[4], o[5], o[6], o[7]);
        } else {
          *reinterpret_cast<uint4*>(base + xlds[j]) = xreg[j];
        }
      }
#pragma unroll
    for (int j = 0; j < WCH; ++j)
      if (WFULL || wok[j]) *reinterpret_cast<uint4*>(base + wlds[j]) = wreg[j];
    if constexpr (MX) {
#pragma unroll
      for (int j = 0; j < SCH; ++j)
        if (SFULL || sok[j]) *reinterpret_cast<uint32_t*>(base + slds[j]) = sreg[j];
    }
  };
  // MFMA step t of a stage: sub-stage s = t / SPS, i = t % SPS; lane group h supplies k = s*128 + h*KG + i*8 .. +8
  auto read_xf = [&](const uint8_t* base, int t, bf16x8_t (&xf)[MFW]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < MFW; ++j)
      xf[j] = *reinterpret_cast<const bf16x8_t*>(base + ((j * WM + mw) * FM + lr) * XPITCH +
                                                  ((t / SPS) * 128 + h * KG + (t % SPS) * 8) * 2);
  };
  // FULL: every row fragment of this wave holds valid rows; the body is then one straight-line block in
  // which the scheduler is told to alternate MFMAs with the dequantisation / LDS reads of the next step.
  auto compute = [&](auto full_c, int buf) __attribute__((always_inline)) {
    constexpr bool FULL = decltype(full_c)::value;
    const uint8_t* base = lds + buf * STAGE;
    const uint8_t* wbase = base + XBYTES + (nw * NFW * FM + lr) * WPITCH;
    constexpr int STEPS = KS * SPS;
    bf16x8_t xf[2][MFW];
    bf16x8_t wf[2][NFW];
    uint32_t wraw[NFW][KG / 8];  // KG e2m1 values of this lane's column (current sub-stage)
    uint32_t sd[NFW];            // the sub-stage's 4 scale bytes of this lane's column
    auto read_w = [&](int sub) __attribute__((always_inline)) {
      if constexpr (MX) {
#pragma unroll
        for (int f = 0; f < NFW; ++f) {
#pragma unroll
          for (int q = 0; q < KG / 32; ++q) {
            const uint4 v = *reinterpret_cast<const uint4*>(wbase + f * FM * WPITCH + sub * 64 + h * (KG / 2) + q * 16);
            wraw[f][4 * q + 0] = v.x;
            wraw[f][4 * q + 1] = v.y;
            wraw[f][4 * q + 2] = v.z;
            wraw[f][4 * q + 3] = v.w;
          }
          sd[f] = *reinterpret_cast<const uint32_t*>(wbase + f * FM * WPITCH + WROW + sub * 4);
        }
      }
    };
    auto make_wf = [&](int t, bf16x8_t (&out)[NFW]) __attribute__((always_inline)) {
      const int sub = t / SPS, i = t % SPS;
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if constexpr (MX) {
          const int blk = h * (KG / 32) + i / 4;  // MX block (of the sub-stage's 4) this step's 8 values lie in
          out[f] = dequant8(wraw[f][i], bits_f32(((sd[f] >> (8 * blk)) & 0xFFu) << 23));
        } else {
          if constexpr (F8) {  // 8 e4m3 -> 8 bf16 (exact)
            const uint2 raw = *reinterpret_cast<const uint2*>(wbase + f * FM * WPITCH + sub * 128 + h * KG + i * 8);
            const bf16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, false);
            const bf16x2_t b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, true);
            const bf16x2_t c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, false);
            const bf16x2_t d2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, true);
            out[f] = bf16x8_t{a[0], a[1], b[0], b[1], c2[0], c2[1], d2[0], d2[1]};
          } else {
            out[f] = *reinterpret_cast<const bf16x8_t*>(wbase + f * FM * WPITCH + (sub * 128 + h * KG + i * 8) * 2);
          }
        }
      }
    };
    read_w(0);
    read_xf(base, 0, xf[0]);
    make_wf(0, wf[0]);
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int cur = t & 1, nxt = cur ^ 1;
      if (t + 1 < STEPS) {
        if ((t + 1) % SPS == 0) read_w((t + 1) / SPS);
        read_xf(base, t + 1, xf[nxt]);
        make_wf(t + 1, wf[nxt]);
      }
#pragma unroll
      for (int j = 0; j < MFW; ++j) {
        if (FULL || j < jcount) {
#pragma unroll
          for (int f = 0; f < NFW; ++f) {
            if constexpr (WK == WK_F16)
              acc[f][j] = FR::mma_f16(wf[cur][f], xf[cur][j], acc[f][j]);
            else
              acc[f][j] = FR::mma(wf[cur][f], xf[cur][j], acc[f][j]);
          }
        }
      }
      if constexpr (FULL) {
        // per MFMA: the share of the next step's VALU work (4 conversions per weight fragment) and LDS reads
        constexpr int NM = MFW * NFW;
        constexpr int VPM = MX ? (4 * NFW + NM - 1) / NM + 1 : 0;
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (m < MFW + (MX ? 0 : NFW)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (VPM) __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
        }
      }
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  auto compute_any = [&](int buf) __attribute__((always_inline)) {
    if (jcount == MFW)
      compute(T_{}, buf);
    else
      compute(F_{}, buf);
  };

  // Pipeline: registers hold stage c+1 (loaded while stage c-1 was computed); at the top of stage c they go
  // to the other LDS buffer, the loads of stage c+2 are issued, then stage c is computed from LDS.
  const int nstages = (K + KC - 1) / KC;
  const int nfull = K / KC;  // stages that lie entirely below K
  auto load_any = [&](int cs) __attribute__((always_inline)) {
    if (cs < nfull)
      load_stage(F_{}, cs * KC);
    else
      load_stage(T_{}, cs * KC);
  };
  load_any(0);
  store_stage(0);
  if (nstages > 1) load_any(1);
  __syncthreads();
  for (int c = 0; c < nstages; ++c) {
    if (c + 1 < nstages) store_stage((c + 1) & 1);
    if (c + 2 < nstages) load_any(c + 2);
    compute_any(c & 1);
    __syncthreads();
  }

  gemm_epilogue<FM, WM, MFW, NFW, SWIGLU, WK == WK_F16>(p, acc, expert, off_m, start_m, eM, n_tile + nw * NFW * FM, n_tile + BN <= N, mw, lr, h);
}

// ------------------------------------------------------------------------------------------------
// MXFP4 weights in the tile-native layout (prefill: block_m 64 / 128)
// ------------------------------------------------------------------------------------------------
// Weight layout (built once per model by the host from the K-contiguous form): per expert, per fragment F of
// 32 output columns, per K-stage s of 128: one 2 KiB block [q:2][lane:64][16 B]; lane = h*32 + lr holds the
// packed e2m1 bytes of column F*32 + lr for k in [s*128 + h*64 + q*32, +32).  Scales: one 128 B block
// [lr:32][4] per (F, s) with the four e8m0 bytes of column lr's stage.  N is padded to 32 and K to 128 with
// zero weights.  A wave owns two column fragments and reads its weights straight from global memory into
// registers (every load instruction fetches 1 KiB contiguous, nothing is shared between waves, so they
// bypass LDS); only the gathered activation rows, which all four waves need, are staged through LDS.
//
// Pipeline per K-stage (8 MFMA steps of k = 16): the MFMAs of step t are interleaved, in program order pinned
// by scheduling barriers, with the LDS reads and e2m1 -> bf16 conversions of step t+1, with the LDS writes of
// the next stage's activations and the global loads of the stage after it.  One workgroup barrier per stage
// sits in step 7, after every wave has fetched its last operands of the current LDS buffer.
//
// G = row groups: with G = 2 the workgroup has eight waves; waves 0-3 own the even 32-row fragments of the tile
// and waves 4-7 the odd ones (same columns), so every SIMD holds two waves whose MFMAs, conversions and memory
// instructions overlap in hardware, while the weights are still fetched from L2 / HBM once per 64*MFW rows.
//
// NFW = column fragments per wave (tile width 128 * NFW): the activation tile is fetched from L2 once per column
// tile, so wider tiles cut the L2 -> L1 traffic, which is what bounds this kernel at prefill shapes.
// WD / XD = depth of the weight register ring (2 or 4) / of the activation staging registers (1 or 2).
// Tail tiles: when at most four of a tile's column fragments lie below N (NFW = 2), wave w multiplies fragment w only
// (its second fragment is loaded but neither converted nor multiplied, and its stores are dropped).
// BLKM = rows of a row block in the ragged metadata (block_m).  A tile processes its block in passes of
// BM = 32 * MFW * G rows; with BLKM = 256 and MFW = 5 an expert of up to 160 rows is ONE tile (weights read
// once, no nearly empty second tile) and only larger blocks take a second pass.
// Slices (experts) whose row and block offsets the persistent MXFP4 prefill kernel keeps in LDS: a tile's coordinates
// then cost LDS reads instead of a chain of dependent global loads.  The host refuses more slices than this.
constexpr int kMetaSlices = 1024;

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
template <int G, int MFW, int NFW, int NFV, bool SWIGLU>
__device__ __forceinline__ void staged_epilogue(const GemmParams& p, f32x16_t (&acc)[NFW][MFW], __amdgpu_buffer_rsrc_t yrsrc, const float* bias_s,
                                                const float* gam_s, const int* dst_s, int ncol_tile, int ncol0, int grp, int lr, int h) {
  const int NOUT = SWIGLU ? p.N / 2 : p.N;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  const uint32_t row_bytes = (uint32_t)(p.y_stride_m * 2);
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const int r = (j * G + grp) * 32 + lr;
    const float g = gam_s[r];
    const int dst = dst_s[r];
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
        const f32x4_t b0 = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 4 * h);
        const f32x4_t b1 = *reinterpret_cast<const f32x4_t*>(bias_s + ncol_tile + f * 32 + 16 * u + 8 + 4 * h);
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

template <int BLKM, int MFW, int NFW, int G, int WD, int XD, bool SWIGLU>
__global__ __launch_bounds__(256 * G) void moe_gemm_mxn_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, NT = 256 * G, BM = MFW * 32 * G, BN = 128 * NFW, KC = 128;
  static_assert((WD == 2 || WD == 4) && (XD == 1 || XD == 2), "ring depths");
  static_assert(BM <= NT && BN <= NT, "one thread per tile row and per tile column fetches the epilogue operands");
  constexpr int XPITCH = KC * 2 + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = BM * 16 / NT;  // 16-byte activation pieces per thread per stage (4 or 8)
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int32_t soffs_s[kMetaSlices], ssize_s[kMetaSlices], boffs_s[kMetaSlices + 1];
  // per-unit operands, two sets used in turn: set (u & 1) holds unit u's epilogue operands and unit u+1's gather indices
  __shared__ __attribute__((aligned(16))) float bias_s[2][BN];
  __shared__ float gam_s[2][BM];
  __shared__ int32_t dst_s[2][BM], gidx_s[2][BM];
  __shared__ int next_tile_s[2];  // slot (n & 1): id of the tile after the next, written during this workgroup's n-th tile

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = wave & 3, grp = wave >> 2;  // column quarter, row group
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;
  const int nfr = (N + 31) >> 5;
  const int xc = tid & 15;
  const int xlds0 = (tid >> 4) * XPITCH + xc * 16;  // activation piece j at xlds0 + j*(NT/16)*XPITCH
  const int grid = (int)gridDim.x;
  const bool ragged = p.slice_sizes != nullptr;
  const int nblk = ragged ? p.block_offs[p.n_slices] : 0;
  const int live = ragged ? nblk * p.grid_n : p.total_tiles;
  if (ragged) {  // (the host admits at most kMetaSlices slices)
    for (int i = tid; i < p.n_slices; i += NT) {
      soffs_s[i] = p.slice_offs[i];
      ssize_s[i] = p.slice_sizes[i];
      boffs_s[i] = p.block_offs[i];
    }
    if (tid == 0) boffs_s[p.n_slices] = nblk;
  }
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);

  // A unit of work = one pass of BM rows over one tile (a row block of one expert x BN columns).  Persistent
  // workgroups walk over tiles either by a static schedule (round r: tile r * grid + remap(block)) or by claiming them
  // (TileClaimer); either way the ids of the next two tiles are known when a tile ends, so that a unit's gather
  // indices and epilogue operands are fetched two and one unit ahead, and its first loads are issued before the
  // previous unit's epilogue arithmetic.
  struct Unit {
    int expert, blk_off, blk_rows, pid_n, start_m, pass_off;
    bool valid;
    bool tail;  // at most four column fragments of the tile lie below N: one per wave (NFW = 2)
  };
  auto tile_unit = [&](int pid) __attribute__((always_inline)) -> Unit {
    Unit u;
    int eM;
    if (ragged) {
      // Tiles are ordered (expert, column tile, row block): the row blocks of one expert that share a column
      // tile get consecutive ids, run at the same time on one XCD and stream the same weights through its L2.
      // The expert is the last slice whose first block is not past block pid / grid_n (empty slices share an
      // offset with their successor): a binary search in the block offsets kept in LDS.
      const int blk = pid / p.grid_n;
      int lo = 0, hi = p.n_slices;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (boffs_s[mid] <= blk) lo = mid; else hi = mid;
      }
      u.expert = lo;
      const int first = boffs_s[lo];
      const int nb = boffs_s[lo + 1] - first;
      const int local = pid - first * p.grid_n;
      u.pid_n = local / nb;
      u.blk_off = (local - u.pid_n * nb) * BLKM;
      u.start_m = soffs_s[lo];
      eM = ssize_s[lo];
    } else {
      u.pid_n = pid % p.grid_n;
      u.expert = 0;
      u.blk_off = (pid / p.grid_n) * BLKM;
      u.start_m = 0;
      eM = p.M;
    }
    u.blk_rows = (eM - u.blk_off) < BLKM ? (eM - u.blk_off) : BLKM;
    u.pass_off = 0;
    u.valid = true;
    u.expert = __builtin_amdgcn_readfirstlane(u.expert);
    u.blk_off = __builtin_amdgcn_readfirstlane(u.blk_off);
    u.blk_rows = __builtin_amdgcn_readfirstlane(u.blk_rows);
    u.pid_n = __builtin_amdgcn_readfirstlane(u.pid_n);
    u.start_m = __builtin_amdgcn_readfirstlane(u.start_m);
    u.tail = NFW == 2 && nfr - u.pid_n * (BN / 32) <= 4;
    return u;
  };
  // the unit after `u`: its next pass, or the first pass of tile `pid_after` (-1: none)
  auto advance = [&](const Unit& u, int pid_after) __attribute__((always_inline)) -> Unit {
    Unit n = u;
    if (u.pass_off + BM < u.blk_rows) {
      n.pass_off = u.pass_off + BM;
    } else if (pid_after >= 0) {
      n = tile_unit(pid_after);
    } else {
      n.valid = false;
    }
    return n;
  };

  // (with the same number of tiles for every workgroup the static schedule is already even, and measured faster)
  // (claiming also needs at least one workgroup per queue, i.e. a grid of 8 or more: a queue's tiles are reached
  // through the workgroups that start on it)
  const bool dyn = p.tile_counters != nullptr && live % grid != 0 && grid >= 8;
  TileClaimer claimer;
  int round0 = 0;
  int pid, pid_next;  // this workgroup's current and next tile id (-1 = none)
  if (dyn) {
    pid = claimer.init(p.tile_counters, live);
    pid_next = pid >= 0 ? claimer.second() : -1;
  } else {
    const int in0 = live < grid ? live : grid;
    pid = (int)blockIdx.x < in0 ? xcd_remap(blockIdx.x, in0) : -1;
    round0 = grid;
    const int in1 = live - round0 < grid ? live - round0 : grid;
    pid_next = (pid >= 0 && (int)blockIdx.x < in1) ? round0 + xcd_remap(blockIdx.x, in1) : -1;
  }
  int n_tile = 0;  // tiles this workgroup has finished
  if (ragged) __syncthreads();

  // ---- per-unit operand addresses: a uniform 64-bit base (scalar registers) plus a 32-bit byte offset per lane, so
  // that they cost one vector register per activation piece and none per weight fragment ----
  uint32_t xoff[XCH];           // byte offset of this thread's row j in x (x spans less than 4 GiB, checked by the host)
  const uint8_t* wbase[NFW];    // uniform: first K-stage of this wave's column fragment f
  const uint8_t* sbase[NFW];
  const uint32_t lane16 = lane * 16, lr4 = lr * 4;
  // gather index (source row of x) of tile row `tid` of unit u, rows past the block's end repeat its last row
  auto unit_gather_index = [&](const Unit& u) __attribute__((always_inline)) -> int {
    int row = u.blk_off + u.pass_off + tid;
    row = row < u.blk_off + u.blk_rows ? row : u.blk_off + u.blk_rows - 1;
    const int srow = u.start_m + row;
    return p.gather ? p.gather[srow] : srow;
  };
  // addresses of unit u from the gather indices staged in gidx_s[set]
  auto unit_pointers = [&](const Unit& u, int set) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      const int r = (tid >> 4) + (NT / 16) * j;
      xoff[j] = (uint32_t)gidx_s[set][r] * (uint32_t)(p.x_stride_m * 2);  // the k offset (incl. this thread's chunk) is added per stage
    }
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      // (tail tiles: fragment nw of the tile is this wave's first, its second lies past N)
      int F = u.pid_n * (BN / 32) + (u.tail ? nw + 4 * f : nw * NFW + f);
      F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
      wbase[f] = p.w + (int64_t)u.expert * p.w_stride_e + (int64_t)F * nst * 2048;
      sbase[f] = p.w_scale + (int64_t)u.expert * p.ws_stride_e + (int64_t)F * nst * 128;
    }
  };
  // Epilogue operands of a unit as thread `tid` fetches them: bias of tile column tid, gate weight and scatter index of
  // tile row tid.  `unit_operands` only issues the loads and keeps the raw bits (anything computed from a loaded value
  // would make the wave wait for it on the spot); `stage_operands` converts them when they go to LDS, a K loop later.
  uint32_t bias_raw = 0, gam_raw = 0;
  int dst_raw = 0, gidx_v = 0;
  auto unit_operands = [&](const Unit& u) __attribute__((always_inline)) {
    const int off_m = u.blk_off + u.pass_off, blk_end = u.blk_off + u.blk_rows;
    if (p.bias) {
      int n = u.pid_n * BN + (tid < BN ? tid : BN - 1);
      n = n < N ? n : N - 1;
      const int64_t i = (int64_t)u.expert * p.bias_stride_e + n;
      bias_raw = p.bias_is_f32 ? static_cast<const uint32_t*>(p.bias)[i] : (uint32_t)static_cast<const uint16_t*>(p.bias)[i];
    }
    int row = off_m + (tid < BM ? tid : BM - 1);
    row = row < blk_end ? row : blk_end - 1;
    const int srow = u.start_m + row;  // row in expert-sorted order
    if (p.gammas) gam_raw = p.gammas_is_f32 ? static_cast<const uint32_t*>(p.gammas)[srow] : (uint32_t)static_cast<const uint16_t*>(p.gammas)[srow];
    if (p.scatter) dst_raw = p.scatter[srow < p.scatter_len ? srow : p.scatter_len - 1];
  };
  auto stage_operands = [&](const Unit& u, int set) __attribute__((always_inline)) {
    // (the index is made opaque so that the LDS addresses are recomputed here instead of being kept in registers)
    int t = tid;
    asm volatile("" : "+v"(t));
    if (t < BN) bias_s[set][t] = p.bias ? bits_f32(p.bias_is_f32 ? bias_raw : bias_raw << 16) : 0.f;
    if (t < BM) {
      const int off_m = u.blk_off + u.pass_off, blk_end = u.blk_off + u.blk_rows;
      const bool ok = off_m + t < blk_end;
      const int srow = u.start_m + off_m + t;
      int dst = srow;
      if (p.scatter) dst = srow < p.scatter_len ? dst_raw : -1;
      gam_s[set][t] = p.gammas ? bits_f32(p.gammas_is_f32 ? gam_raw : gam_raw << 16) : 1.0f;
      dst_s[set][t] = ok ? dst : -1;
      gidx_s[set][t] = gidx_v;
    }
  };

  typename FR::acc_t acc[NFW][MFW];
  // activation staging registers, XD stages deep: stage c writes X(c+1) from slot (c+1) % XD to LDS and refills it
  // with X(c+1+XD).  (Native vectors: arrays of the HIP uint4 struct were left in scratch memory here.)
  u32x4_t xreg[XD][XCH];
  // weight register ring: stage c uses slot c % WD, loads run WD-1 stages ahead
  u32x4_t wraw[WD][NFW][2];
  uint32_t sd[WD][NFW];
  bf16x8_t xf[2][MFW];
  bf16x8_t wf[2][NFW];

  // Loads are unconditional (no divergent control flow inside the pipeline): rows past the tile's last
  // valid row re-read that row, k past K re-reads the row's last 8 values (the padded weights there are
  // zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s, int slot) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 8;
    k0 = k0 < K - 8 ? k0 : K - 8;
    xreg[slot][j] = *reinterpret_cast<const u32x4_t*>(p.x + (xoff[j] + (uint32_t)(k0 * 2)));
  };
  auto store_x_piece = [&](int j, int buf, int slot) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * (NT / 16) * XPITCH) = xreg[slot][j];
  };
  auto load_w = [&](auto par_c, int s) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      wraw[PAR][f][0] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + lane16);
      wraw[PAR][f][1] = *reinterpret_cast<const u32x4_t*>(wbase[f] + (int64_t)s * 2048 + 1024 + lane16);
      sd[PAR][f] = *reinterpret_cast<const uint32_t*>(sbase[f] + (int64_t)s * 128 + lr4);
    }
  };
  // operands of step t of the stage held in LDS buffer `buf` / weight registers PAR
  auto read_xf = [&](int buf, int t, int j, bf16x8_t (&out)[MFW]) __attribute__((always_inline)) {
    out[j] = *reinterpret_cast<const bf16x8_t*>(lds + buf * XBYTES + ((j * G + grp) * FM + lr) * XPITCH + h * 128 + t * 16);
  };
  // The empty volatile asm statements pin the conversion between the MFMAs of its slot: without them the
  // (side-effect free) conversions drift to the start of the next step and serialise with the MFMAs.
  auto make_wf = [&](auto par_c, int t, int f, bf16x8_t (&out)[NFW]) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value;
    const u32x4_t v = wraw[PAR][f][t >> 2];
    uint32_t raw = (t & 3) == 0 ? v.x : (t & 3) == 1 ? v.y : (t & 3) == 2 ? v.z : v.w;
    asm volatile("" : "+v"(raw));
    const uint32_t sbyte = (sd[PAR][f] >> (8 * (t >> 2))) >> (16 * h);  // MX block h*2 + t/4 of the stage
    u32x4_t r = __builtin_bit_cast(u32x4_t, dequant8(raw, bits_f32((sbyte & 0xFFu) << 23)));
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
    out[f] = __builtin_bit_cast(bf16x8_t, r);
  };

  template_int<0> S0;
  template_int<1> S1;
  template_int<2> S2;
  template_int<3> S3;

  // One K-stage.  NJ = row fragments with valid rows (compile-time so the MFMA list is straight-line code);
  // only the 2*NJ activation pieces per thread that cover those fragments are staged.  WS = weight ring slot
  // of this stage (= c % WD); the activation LDS buffer is WS & 1.
  auto stage = [&](auto nj_c, auto gi_c, auto nf_c, auto ws_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int NFV = decltype(nf_c)::value;  // column fragments of this wave that are multiplied (the loads always cover NFW)
    constexpr int WS4 = decltype(ws_c)::value;  // c % 4
    constexpr int PAR = WS4 & 1;
    using WSC = template_int<WS4 % WD>;                // this stage's weights
    using WSN = template_int<(WS4 + 1) % WD>;          // next stage's weights
    using WSL = template_int<(WS4 + WD - 1) % WD>;     // slot to refill: stage c + WD - 1
    constexpr int XS = (WS4 + 1) % XD;                 // activation register slot holding X(c+1)
    constexpr int WLOAD_STEP = WD == 2 ? 0 : 4;        // the refilled slot was last read in step 6 of stage c-1
    constexpr int GI = decltype(gi_c)::value;  // this wave's row group
    constexpr int NM = NJ * NFV;
    // pieces to stage: a piece covers 16 rows (G = 1) or 32 rows (G = 2); with G = 2 the tile has 2*NJ - 1 or 2*NJ
    // (group 0), 2*NJ or 2*NJ + 1 (group 1) fragments with valid rows, and the larger count is staged
    constexpr int NP = G == 1 ? 2 * NJ : (2 * NJ + GI < XCH ? 2 * NJ + GI : XCH);
    constexpr int PPS = (NP + 3) / 4;    // per step, during steps 0..3
    constexpr int NOPS = NJ + NFV + 4;   // NJ LDS reads, NFV conversions, three staging slots, the weight loads
    static_for<0, 8>([&](auto t_c) __attribute__((always_inline)) {
      constexpr int t = decltype(t_c)::value;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o == NJ + NFV + 3) {
          if constexpr (t == WLOAD_STEP) load_w(WSL{}, c + WD - 1);
        } else if constexpr (t < 7) {
          if constexpr (o < NJ) {
            read_xf(PAR, t + 1, o, xf[nxt]);
          } else if constexpr (o < NJ + NFV) {
            make_wf(WSC{}, t + 1, o - NJ, wf[nxt]);
          } else if constexpr (t < 4) {
            // next stage's activations: registers -> LDS, then refill the registers for a later stage
            constexpr int half = o - NJ - NFV;
            constexpr int j = t * PPS + half;
            if constexpr (half < PPS && j < NP) {
              store_x_piece(j, PAR ^ 1, XS);
              load_x_piece(j, c + 1 + XD, XS);
            }
          }
        } else {
          if constexpr (o < NJ) {
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
          } else if constexpr (o < NJ + NFV) {
            make_wf(WSN{}, 0, o - NJ, wf[nxt]);
          }
        }
      };
      if constexpr (NM == 0) {
        // a wave without valid rows still stages its share of the activations and joins the barriers
        if constexpr (t == 7) {
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<0, NOPS>(op);
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFV, f = m % NFV;
        acc[f][j] = FR::mma(wf[cur][f], xf[cur][j], acc[f][j]);
        if constexpr (t == 7 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 6) and written its share
          // of the next one (steps 0..3)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        // ops are dealt as evenly as possible: slot m runs ops [m*NOPS/NM, (m+1)*NOPS/NM)
        static_for<(m * NOPS) / (NM ? NM : 1), ((m + 1) * NOPS) / (NM ? NM : 1)>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  // Stage 0 of a unit (activations of every piece, weights): issued before the previous unit's epilogue arithmetic.
  auto first_loads = [&]() __attribute__((always_inline)) {
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0, 0); });
    __builtin_amdgcn_sched_barrier(0);
    load_w(S0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  int up = 0;             // operand set of the current unit
  Unit cur_unit;          // the unit being computed
  int resolve_slot = -1;  // thread 0 writes the claimed tile id into next_tile_s[resolve_slot] before the first barrier
  auto run = [&](auto nj_c, auto gi_c, auto nf_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int GI = decltype(gi_c)::value;
    constexpr int NFV = decltype(nf_c)::value;
    constexpr int NP = G == 1 ? 2 * NJ : (2 * NJ + GI < XCH ? 2 * NJ + GI : XCH);
    // Prologue: finish stage 0 (its loads were issued by first_loads before the previous unit's epilogue).  The order
    // of the loads left in flight (activations, then weights, of stage 1, then of stage 2) is pinned to the order the
    // steady state leaves them in at the top of a stage: the compiler's wait counts at the loop header are the merge
    // of both paths, and any mismatch makes every iteration wait for the loads it has just issued.
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1, 1 % XD); });
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (WD == 4) {
      load_w(S1, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (XD == 2) {
      static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 2, 0); });
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (WD == 4) {
      load_w(S2, 2);
      __builtin_amdgcn_sched_barrier(0);
    }
    // what was fetched during the previous unit's epilogue goes to LDS: this unit's epilogue operands and the next
    // unit's gather indices (set `up`; its last readers were the epilogue and the address set-up two units back)
    stage_operands(cur_unit, up);
    // the claim issued before the previous epilogue has had that long to travel
    if (resolve_slot >= 0 && tid == 0) next_tile_s[resolve_slot] = claimer.resolve();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { read_xf(0, 0, decltype(jc)::value, xf[0]); });
    static_for<0, NFV>([&](auto fc) __attribute__((always_inline)) { make_wf(S0, 0, decltype(fc)::value, wf[0]); });
    __builtin_amdgcn_sched_barrier(0);
    // all stages of a group always run inside the loop: a path that skips some and returns to the loop header
    // would again make the header's wait counts cover the loads just issued
    int c = 0;
    for (; c + 3 < nst; c += 4) {
      stage(nj_c, gi_c, nf_c, S0, c);
      stage(nj_c, gi_c, nf_c, S1, c + 1);
      stage(nj_c, gi_c, nf_c, S2, c + 2);
      stage(nj_c, gi_c, nf_c, S3, c + 3);
    }
    if (c < nst) stage(nj_c, gi_c, nf_c, S0, c);
    if (c + 1 < nst) stage(nj_c, gi_c, nf_c, S1, c + 1);
    if (c + 2 < nst) stage(nj_c, gi_c, nf_c, S2, c + 2);
  };
  auto dispatch = [&](auto gi_c, auto nf_c, int nj) __attribute__((always_inline)) {
    constexpr int GI = decltype(gi_c)::value;
    if constexpr (GI == 1) {
      if (nj == 0) {
        run(template_int<0>{}, gi_c, nf_c);
        return;
      }
    }
    static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
      if (nj == decltype(n_c)::value) run(n_c, gi_c, nf_c);
    });
  };
  // (tail tiles multiply one fragment per wave)
  auto dispatch_nf = [&](auto gi_c, bool tail, int nj) __attribute__((always_inline)) {
    if constexpr (NFW == 2) {
      if (tail) {
        dispatch(gi_c, template_int<1>{}, nj);
        return;
      }
    }
    dispatch(gi_c, template_int<NFW>{}, nj);
  };

  if (pid >= 0) {
    Unit& cur = cur_unit;
    cur = tile_unit(pid);
    Unit nxt = advance(cur, pid_next);
    // the first unit has nothing to hide behind: gather indices, addresses, operands, first loads
    if (tid < BM) gidx_s[1][tid] = unit_gather_index(cur);
    __syncthreads();
    unit_pointers(cur, 1);
    unit_operands(cur);
    if (nxt.valid && tid < BM) gidx_v = unit_gather_index(nxt);
    if (dyn && pid_next >= 0) {
      claimer.issue();  // the tile after the next
      resolve_slot = 0;
    }
    first_loads();
    for (;;) {
#pragma unroll
      for (int f = 0; f < NFW; ++f)
#pragma unroll
        for (int j = 0; j < MFW; ++j)
#pragma unroll
          for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;
      const int rows = (cur.blk_rows - cur.pass_off) < BM ? (cur.blk_rows - cur.pass_off) : BM;
      const int nfrag_m = (rows + FM - 1) / FM;  // row fragments that hold valid rows (1..MFW*G)
      const int nj = (nfrag_m - grp + G - 1) / G;  // those of this wave: tile fragments grp, grp + G, ...
      if constexpr (G == 2) {
        if (grp == 1)
          dispatch_nf(template_int<1>{}, cur.tail, nj);
        else
          dispatch_nf(template_int<0>{}, cur.tail, nj);
      } else {
        dispatch_nf(template_int<0>{}, cur.tail, nj);
      }
      resolve_slot = -1;

      // ---- before this unit's epilogue: everything the next units need from memory ----
      const int wcol = cur.tail ? nw * FM : nw * NFW * FM;  // this wave's first column in the tile
      const int ncol0 = cur.pid_n * BN + wcol;
      const bool cur_tail = cur.tail;
      Unit nxt2 = nxt;
      if (nxt.valid) {
        if (cur.pass_off + BM >= cur.blk_rows) {
          // the next unit opens a new tile; the tile after it was claimed during this tile's first prologue (or
          // follows statically)
          pid = pid_next;
          ++n_tile;
          if (dyn) {
            pid_next = __builtin_amdgcn_readfirstlane(next_tile_s[(n_tile - 1) & 1]);
          } else {
            round0 += grid;
            const int in_round = live - round0 < grid ? live - round0 : grid;
            pid_next = (int)blockIdx.x < in_round ? round0 + xcd_remap(blockIdx.x, in_round) : -1;
          }
          if (dyn && pid_next >= 0) {
            claimer.issue();
            resolve_slot = n_tile & 1;
          }
        }
        nxt2 = advance(nxt, pid_next);
        // (these loads and the claim come BEFORE the next unit's first loads: the number of them in flight differs
        // from path to path, and only what is issued after a load makes the wait for that load inexact)
        unit_operands(nxt);
        if (nxt2.valid && tid < BM) gidx_v = unit_gather_index(nxt2);
        __builtin_amdgcn_sched_barrier(0);
        unit_pointers(nxt, up);
        first_loads();
      }
      if (NFW == 2 && cur_tail)
        staged_epilogue<G, MFW, NFW, 1, SWIGLU>(p, acc, yrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, grp, lr, h);
      else
        staged_epilogue<G, MFW, NFW, NFW, SWIGLU>(p, acc, yrsrc, bias_s[up], gam_s[up], dst_s[up], wcol, ncol0, grp, lr, h);
      if (!nxt.valid) break;
      cur = nxt;
      nxt = nxt2;
      up ^= 1;
    }
  }
  if (dyn) claimer.finish();
}

// ------------------------------------------------------------------------------------------------
// MXFP4 weights in the tile-native layout, decode shapes (block_m 16 / 32): a pure weight stream
// ------------------------------------------------------------------------------------------------
// A few rows per expert: the kernel is bound by reading each active expert's weights once.  Every wave works
// alone (no LDS, no barrier): it owns one 32-column weight fragment of one row block, streams the fragment's
// K-stages through a four-deep register ring (8 KiB in flight per wave, twelve to sixteen waves per CU), reads its
// rows' activations straight from L2 through a ring of the same depth (each lane 64 contiguous bytes per stage;
// one stage ahead left their latency exposed), and issues 16x16x32 MFMAs
// transposed like the prefill kernel (lane = column, 4 k-groups).  Within a stage lane group kg owns
// k in [kg*32, kg*32 + 32): exactly one MX block and one 16-byte piece of the tiled layout.
// Epilogue of the decode kernel with the top-k combine fused behind the scatter (the reference runs `reduce` over the k
// rows of every token as a launch of its own, reduce.py:1143-1165).  The k rows of token t are written by up to k
// different waves, anywhere on the chip; each counts itself in at counter (t, fragment) once its rows have reached
// memory, and the wave that arrives last sums the k rows in their order j = 0..k-1 in fp32, exactly as the
// stand-alone kernel does, writes the token's row of the result and clears the counter for the next launch.
// The eight XCDs have an L2 each, so rows that another XCD will read go around it: stores and loads of y carry the
// sc0 sc1 cache policy (write-through to memory / read from memory) and the counter is a device-scope atomic; the
// alternative, a device-scope release fence per wave, writes back and invalidates a whole L2 each time and more than
// doubled the kernel's time.  acc[g][j][i]: sub-fragment g (columns F*32 + g*16 + kg*4 + i), row fragment j.
// Operands of the combine epilogue that do not depend on the accumulators; the kernel fetches them before its K loop
// so that their latency is not part of every wave's tail.
template <int MR, int NFD>
struct CombineOperands {
  float gam[MR];
  int dst[MR];          // destination row (flat position t * k + j) or -1
  float b4[NFD][2][4];  // bias of the lane's columns
};

template <int MR, int NFD>
__device__ __forceinline__ CombineOperands<MR, NFD> load_combine_operands(const GemmParams& p, int expert, int off_m, int start_m, int eM,
                                                                          const int (&F)[NFD], int lr, int kg) {
  CombineOperands<MR, NFD> o;
  const int N = p.N;
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = F[fd] * 32 + g * 16 + kg * 4 + i;
        o.b4[fd][g][i] = (p.bias && n < N) ? load_scalar(p.bias, (int64_t)expert * p.bias_stride_e + n, p.bias_is_f32) : 0.f;
      }
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int row = off_m + j * 16 + lr;
    const bool ok = row < eM;
    const int srow = start_m + (ok ? row : eM - 1);
    o.gam[j] = p.gammas ? load_scalar(p.gammas, srow, p.gammas_is_f32) : 1.0f;
    const int dst = srow < p.scatter_len ? p.scatter[srow] : -1;
    o.dst[j] = ok ? dst : -1;
  }
  return o;
}

// The NFD fragments of a wave go through every step together (all stores, one wait, all counters, all loads), so the
// chain of memory round trips at the end of a wave is as long for two fragments as for one.
template <int MR, int NFD>
__device__ __forceinline__ void combine_epilogue(const GemmParams& p, f32x4_t (&acc)[NFD][2][MR], const CombineOperands<MR, NFD>& o,
                                                 const int (&F)[NFD], const bool (&live_f)[NFD], int nfr, int lr, int kg) {
  constexpr int kThrough = 1 | 16;  // aux bits of the buffer instructions: sc0 | sc1
  const int N = p.N, k = p.combine_k;
  const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.y_bytes, 0x00020000);
  const uint32_t row_bytes = (uint32_t)(p.y_stride_m * 2);
  int token[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int dst = o.dst[j];
    const float gam = o.gam[j];
    token[j] = dst >= 0 ? dst / k : -1;
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const int n0 = F[fd] * 32 + g * 16 + kg * 4;
        const u32x2_t w = {pack_bf16x2((acc[fd][g][j][0] + o.b4[fd][g][0]) * gam, (acc[fd][g][j][1] + o.b4[fd][g][1]) * gam),
                           pack_bf16x2((acc[fd][g][j][2] + o.b4[fd][g][2]) * gam, (acc[fd][g][j][3] + o.b4[fd][g][3]) * gam)};
        const uint32_t off = (live_f[fd] && dst >= 0 && n0 < N) ? (uint32_t)dst * row_bytes + (uint32_t)n0 * 2u : kDroppedStore;
        __builtin_amdgcn_raw_buffer_store_b64(w, yrsrc, off, 0, kThrough);
      }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows have reached memory before it is counted
  bool last[MR][NFD];
#pragma unroll
  for (int j = 0; j < MR; ++j)
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd) {
      int seen = -1;
      if (kg == 0 && token[j] >= 0 && live_f[fd])
        seen = __hip_atomic_fetch_add(&p.combine_counters[(int64_t)token[j] * nfr + F[fd]], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      seen = __shfl(seen, lr);  // the row's four lanes (lr, lr + 16, ...) share lane lr's count
      last[j][fd] = token[j] >= 0 && live_f[fd] && seen == k - 1;
    }
  // (the loads below depend on the atomics' results, so they cannot be issued before those have been performed)
#pragma unroll
  for (int j = 0; j < MR; ++j)
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd) {
      const uint32_t base = last[j][fd] ? (uint32_t)(token[j] * k) * row_bytes : kDroppedStore;
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const int n0 = F[fd] * 32 + g * 16 + kg * 4;
        float sum[4] = {0.f, 0.f, 0.f, 0.f};
        for (int jj = 0; jj < k; ++jj) {
          const uint32_t off = (last[j][fd] && n0 < N) ? base + (uint32_t)jj * row_bytes + (uint32_t)n0 * 2u : kDroppedStore;
          const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(yrsrc, off, 0, kThrough);  // out-of-range lanes read zero
          sum[0] += bits_f32(v.x << 16);
          sum[1] += bits_f32(v.x & 0xFFFF0000u);
          sum[2] += bits_f32(v.y << 16);
          sum[3] += bits_f32(v.y & 0xFFFF0000u);
        }
        if (last[j][fd] && n0 < N) {
          uint16_t* out = p.combine_out + (int64_t)token[j] * p.combine_stride + n0;
          if (n0 + 4 <= N && (p.combine_stride & 3) == 0) {
            *reinterpret_cast<uint2*>(out) = make_uint2(pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3]));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n0 + i < N) out[i] = f32_to_bf16_bits(sum[i]);
          }
        }
      }
      if (last[j][fd] && kg == 0)
        __hip_atomic_store(&p.combine_counters[(int64_t)token[j] * nfr + F[fd]], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int MR, int NFD, bool SWIGLU>
__global__ __launch_bounds__(256) void moe_gemm_mxd_kernel(const GemmParams p) {
  typedef Frag<16> FR;
  constexpr int WDD = 4, XDD = 4;  // ring depths (stages) of the weight / activation registers (both run 3 stages ahead)
  __shared__ float red[3][NFD * 2 * MR * 4][64];  // K-split partial sums of waves 1..3
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, kg = lane >> 4;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;
  const int nfr = (N + 31) >> 5;
  // A wave owns NFD neighbouring 32-column fragments of one row block: the activations it fetches (twice the bytes of a
  // fragment's weights per stage) then feed NFD fragments' MFMAs.
  const int nslot = (nfr + NFD - 1) / NFD;  // fragment groups per row block

  // K-split: when few tiles are live (a handful of active experts), 2 or 4 waves share a fragment group and take
  // every 2nd / 4th K-stage each, so that enough loads are in flight to cover the HBM latency.  The factor is
  // derived on the device from the live block count (the host never reads it) and is uniform over the grid;
  // the grid is launched for the largest factor and the surplus workgroups leave at once.
  const int nblk = p.slice_sizes ? p.block_offs[p.n_slices] : p.total_tiles;
  const int frag_tiles = nblk * nslot;  // (row block, fragment group) pairs = waves at split 1
  const int ksplit = frag_tiles <= 1024 ? 4 : (frag_tiles <= 2048 ? 2 : 1);
  const int fpw = 4 / ksplit;                        // fragment groups per workgroup
  const int grid_n = (nslot + fpw - 1) / fpw;        // workgroups per row block
  // Workgroups go round-robin to the 8 XCDs.  With the row blocks a multiple of 8 workgroups apart, the workgroups that
  // read one weight fragment for the different row blocks of an expert (an expert with more rows than a block holds)
  // land on ONE XCD, close together in time, and share the fragment through its L2 instead of fetching it again.
  const int grid_n8 = (grid_n + 7) & ~7;
  if ((int)blockIdx.x >= nblk * grid_n8) return;
  const int pid_n = blockIdx.x % grid_n8, pid_m = blockIdx.x / grid_n8;
  if (pid_n >= grid_n) return;
  const int kslice = wave % ksplit;
  int expert, off_m, start_m, eM;
  if (p.slice_sizes) {
    const int sched = p.block_sched[pid_m];
    expert = sched & 0xFFFF;
    off_m = (sched >> 16) * (MR * 16);
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    expert = 0;
    off_m = pid_m * (MR * 16);
    start_m = 0;
    eM = p.M;
  }
  const int slot = pid_n * fpw + wave / ksplit;  // this wave's fragment group
  const bool live_wave = slot < nslot;
  int F[NFD];
  bool live_f[NFD];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    const int f = (live_wave ? slot : nslot - 1) * NFD + fd;
    live_f[fd] = live_wave && f < nfr;
    F[fd] = f < nfr ? f : nfr - 1;
  }
  const int rows = (eM - off_m) < MR * 16 ? (eM - off_m) : MR * 16;
  const int nj = (rows + 15) >> 4;  // row fragments with valid rows (1..MR)
  // this wave's stages: kslice, kslice + ksplit, ...
  const int my_nst = (nst - kslice + ksplit - 1) / ksplit;

  // weights: sub-fragment g holds columns F*32 + g*16 + lr; this lane's piece of a stage is k-block kg
  const uint8_t* wbase[NFD];
  const uint8_t* sbase[NFD];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    wbase[fd] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F[fd] * nst * 2048 + (kg & 1) * 1024 + ((kg >> 1) * 32 + lr) * 16;
    sbase[fd] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)F[fd] * nst * 128 + lr * 4;
  }
  // activations: row j*16 + lr, 64 bytes per stage at k offset kg*32
  const uint8_t* xptr[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    int row = off_m + j * 16 + lr;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m * 2;
  }

  typename FR::acc_t acc[NFD][2][MR];
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int j = 0; j < MR; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[fd][g][j][i] = 0.f;

  u32x4_t wr[WDD][NFD][2];
  uint32_t sr[WDD][NFD][2];
  u32x4_t xr[XDD][MR][4];

  // `i` counts this wave's own stages; the global stage is kslice + i*ksplit (clamped: surplus loads re-read
  // the last stage and are never used)
  auto load_w = [&](auto slot_c, int i) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    int s = kslice + i * ksplit;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        wr[SL][fd][g] = *reinterpret_cast<const u32x4_t*>(wbase[fd] + (int64_t)s * 2048 + g * 256);
        sr[SL][fd][g] = *reinterpret_cast<const uint32_t*>(sbase[fd] + (int64_t)s * 128 + g * 64);
      }
  };
  auto load_x = [&](auto slot_c, int i) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    const int s = kslice + i * ksplit;
#pragma unroll
    for (int j = 0; j < MR; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int k0 = s * 128 + kg * 32 + t * 8;
        k0 = k0 < K - 8 ? k0 : K - 8;  // past K the padded weights are zero; any finite activation will do
        xr[SL][j][t] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0 * 2);
      }
  };
  auto compute = [&](auto wslot_c, auto xslot_c) __attribute__((always_inline)) {
    constexpr int WS = decltype(wslot_c)::value;
    constexpr int XS = decltype(xslot_c)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8_t wf[NFD][2];
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const u32x4_t v = wr[WS][fd][g];
          const uint32_t raw = t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
          wf[fd][g] = dequant8(raw, bits_f32(((sr[WS][fd][g] >> (8 * kg)) & 0xFFu) << 23));
        }
#pragma unroll
      for (int j = 0; j < MR; ++j) {
        if (j < nj) {
          const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, xr[XS][j][t]);
#pragma unroll
          for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
            for (int g = 0; g < 2; ++g) acc[fd][g][j] = FR::mma(wf[fd][g], xf, acc[fd][g][j]);
        }
      }
    }
  };

  CombineOperands<MR, NFD> cops;
  bool combine = false;
  if constexpr (!SWIGLU) {
    combine = p.combine_k > 0;
    if (combine && live_wave && kslice == 0) cops = load_combine_operands<MR, NFD>(p, expert, off_m, start_m, eM, F, lr, kg);
  }
  if (live_wave) {
    // prologue: fill the rings in the order the steady state leaves them (weights run WDD-1 stages ahead,
    // activations XDD-1)
    static_for<0, WDD - 1>([&](auto c_c) __attribute__((always_inline)) {
      constexpr int c = decltype(c_c)::value;
      load_w(c_c, c);
      if constexpr (c < XDD - 1) load_x(c_c, c);
    });
    int c = 0;
    for (; c + WDD - 1 < my_nst; c += WDD) {
      static_for<0, WDD>([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        load_w(template_int<(i + WDD - 1) % WDD>{}, c + i + WDD - 1);
        load_x(template_int<(i + XDD - 1) % XDD>{}, c + i + XDD - 1);
        compute(i_c, template_int<i % XDD>{});
      });
    }
    static_for<0, WDD - 1>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if (c + i < my_nst) {
        load_x(template_int<(i + XDD - 1) % XDD>{}, c + i + XDD - 1);
        compute(i_c, template_int<i % XDD>{});
      }
    });
  }
  if (ksplit > 1) {
    // sum the K-slices of a fragment group in the wave with kslice 0 (through LDS), which then runs the epilogue
    if (kslice != 0) {
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int j = 0; j < MR; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave - 1][((fd * 2 + g) * MR + j) * 4 + i][lane] = acc[fd][g][j][i];
    }
    __syncthreads();
    if (kslice != 0) return;
    for (int o = 1; o < ksplit; ++o)
#pragma unroll
      for (int fd = 0; fd < NFD; ++fd)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int j = 0; j < MR; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[fd][g][j][i] += red[wave + o - 1][((fd * 2 + g) * MR + j) * 4 + i][lane];
  }
  if constexpr (!SWIGLU) {
    if (combine) {
      if (live_wave) combine_epilogue<MR, NFD>(p, acc, cops, F, live_f, nfr, lr, kg);
      return;
    }
  }
#pragma unroll
  for (int fd = 0; fd < NFD; ++fd) {
    if (!live_f[fd]) continue;
    gemm_epilogue<16, 1, MR, 2, SWIGLU>(p, acc[fd], expert, off_m, start_m, eM, F[fd] * 32, F[fd] * 32 + 32 <= N, 0, lr, kg);
  }
}

// ------------------------------------------------------------------------------------------------
// e4m3 weights in a tile-native layout x e4m3 activations (prefill): FP8 MFMA, no conversion in the loop
// ------------------------------------------------------------------------------------------------
// Weight layout (built once per model by the host from the K-contiguous form): per expert, per fragment F of 32
// output columns (N padded to 32), per K-block s of 128 (K padded to 256 with zero weights, so the number of
// blocks is even): one 4 KiB block [q:4][lane:64][16 B]; lane = h*32 + lr holds the e4m3 bytes of column
// F*32 + lr for k in [s*128 + (q/2)*64 + h*32 + (q%2)*16, +16): pieces 2t and 2t+1 of a lane are the 32 consecutive
// bytes it feeds to the v_mfma_f32_32x32x64_f8f6f4 of K-step t.  The activation rows (gathered, one byte per
// element) are staged through LDS and read back as the same 32 consecutive bytes per lane, so both operands put
// the same k in the same byte position whatever order the instruction sums them in.  Per-row and per-column
// fp32 scales, bias, activation and gate weight are applied by the shared epilogue.
//
// Structure as in the MXFP4 prefill kernel: four waves, each owning NFW column fragments whose weights go
// global memory -> register double buffer -> MFMA, all sharing the MFW row fragments of the tile through an LDS
// double buffer; persistent grid with XCD-aware rounds and (expert, column tile, row block) tile order.  A stage
// is 256 bytes of K = four K-steps of 64, one workgroup barrier per stage (in step 3); the 64 memory instructions
// of a stage (LDS reads of the next step's activations, LDS writes of the next stage's activations with the
// refill of their staging registers, weight loads of the next stage) are dealt two or three to each of the 32
// MFMA slots: a slot that issues many loads back to back holds up the next MFMA.
template <int BLKM, int MFW, int NFW, bool SWIGLU>
__global__ __launch_bounds__(256) void moe_gemm_f8n_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, BM = MFW * 32, BN = 128 * NFW, KC = 256, NS = 4;
  constexpr int XPITCH = KC + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = 2 * MFW;  // 16-byte activation pieces per thread per stage
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);  // column quarter of the tile
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;  // stages of 256 (two 4 KiB weight blocks per column fragment each)
  const int live = p.slice_sizes ? p.block_offs[p.n_slices] * p.grid_n : p.total_tiles;
  __shared__ int next_tile_s[2];  // written by thread 0 before a tile's first barrier: the id of the tile after it
  int tile_par = 0, n_tile = 0;
  // (claiming needs at least one workgroup per XCD queue: a queue's tiles are reached through the workgroups that
  // start on it.  With many rounds, or tiles that divide evenly among the workgroups, the static rounds are kept: a
  // partly filled last round then costs little, while tiles that start together walk K in step and find each other's
  // operands in the XCD's L2 — 4 % faster at 8192 tokens x top-2 of 8 experts, 56 rounds.)
  const bool dyn = p.tile_counters != nullptr && gridDim.x >= 8 && live % (int)gridDim.x != 0 && live < 32 * (int)gridDim.x;
  TileClaimer claimer;
  int pid = claimer.init(p.tile_counters, live), round0 = 0;
  // (dynamic: a workgroup whose queue is shorter than its first index gets no tile at all, which only happens when
  // there are fewer tiles than workgroups; its first two tiles are fixed, later ones are claimed)
  const int pid_second = claimer.second();
  if (!dyn) {
    const int in_round0 = live < (int)gridDim.x ? live : (int)gridDim.x;
    pid = (int)blockIdx.x < in_round0 ? xcd_remap(blockIdx.x, in_round0) : -1;
  }
  while (pid >= 0) {
  const bool claim_now = dyn && (n_tile >= 1 || pid_second < 0);
  if (claim_now) claimer.issue();  // the next tile's claim travels while this tile's first loads do
  int expert, blk_off, start_m, eM, pid_n;
  if (p.slice_sizes) {
    expert = p.block_sched[pid / p.grid_n] & 0xFFFF;
    const int first = p.block_offs[expert];
    const int nb = p.block_offs[expert + 1] - first;
    const int local = pid - first * p.grid_n;
    pid_n = local / nb;
    blk_off = (local - pid_n * nb) * BLKM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    pid_n = pid % p.grid_n;
    expert = 0;
    blk_off = (pid / p.grid_n) * BLKM;
    start_m = 0;
    eM = p.M;
  }
  const int blk_rows = (eM - blk_off) < BLKM ? (eM - blk_off) : BLKM;
  for (int pass_off = 0; pass_off < blk_rows; pass_off += BM) {
  const int off_m = blk_off + pass_off;
  const int rows = (blk_rows - pass_off) < BM ? (blk_rows - pass_off) : BM;
  const int nj = (rows + FM - 1) / FM;  // row fragments that hold valid rows (1..MFW)

  // ---- activation staging: piece j of this thread = row 16 j + tid/16, 16-byte chunk tid%16 of the stage ----
  const int xc = tid & 15;
  const uint8_t* xptr[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int row = off_m + (tid >> 4) + 16 * j;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m;
  }
  const int xlds0 = (tid >> 4) * XPITCH + xc * 16;  // piece j at xlds0 + j*16*XPITCH

  const int nfr = (N + 31) >> 5;
  const uint8_t* wptr[NFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f) {
    int F = pid_n * (BN / 32) + nw * NFW + f;
    F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
    wptr[f] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F * nst * 8192 + lane * 16;
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  u32x4_t xreg[XCH];
  i32x8_t wreg[2][NFW][NS];  // [stage parity][column fragment][K-step]
  i32x8_t xf[2][MFW];        // [K-step parity][row fragment]

  // Loads are unconditional: rows past the last valid row re-read it, k past K re-reads the row's last 16 bytes
  // (the padded weights there are zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 16;
    k0 = k0 < K - 16 ? k0 : K - 16;
    xreg[j] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0);
  };
  auto store_x_piece = [&](int j, int buf) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 16 * XPITCH) = xreg[j];
  };
  // weights of K-step t of column fragment f, stage s, into register set SL
  auto load_w = [&](auto slot_c, int f, int t, int s) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    s = s < nst ? s : nst - 1;
    const uint8_t* a = wptr[f] + (int64_t)s * 8192 + t * 2048;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 1024);
    wreg[SL][f][t] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_xf = [&](int buf, int t, int j, i32x8_t (&out)[MFW]) __attribute__((always_inline)) {
    const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + t * 64 + h * 32;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 16);
    out[j] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  template_int<0> S0;
  template_int<1> S1;

  // One stage.  NJ = row fragments with valid rows; PAR = c & 1 = LDS buffer and weight register set.
  // Ops of step t: NJ reads of step t+1's activation fragments (step 3: the next stage's step 0, after the
  // barrier), in steps 0..2 the staging of the next stage's activations (2 NJ pieces over three steps) and in
  // every step two (fragment, K-step) pairs of the next stage's weights.
  auto stage = [&](auto nj_c, auto par_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int PAR = decltype(par_c)::value;
    using NXT = template_int<PAR ^ 1>;
    constexpr int NM = NJ * NFW;
    constexpr int NP = 2 * NJ;
    constexpr int PPS = (NP + 2) / 3;          // pieces staged per step during steps 0..2
    constexpr int WPS = (NFW * NS + NS - 1) / NS;  // weight (fragment, K-step) pairs loaded per step
    constexpr int NOPS = NJ + PPS + WPS;
    static_for<0, NS>([&](auto t_c) __attribute__((always_inline)) {
      constexpr int t = decltype(t_c)::value;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o < NJ) {
          if constexpr (t < NS - 1)
            read_xf(PAR, t + 1, o, xf[nxt]);
          else
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
        } else if constexpr (o < NJ + PPS) {
          constexpr int j = t * PPS + (o - NJ);
          if constexpr (t < NS - 1 && j < NP) {
            store_x_piece(j, PAR ^ 1);
            load_x_piece(j, c + 2);
          }
        } else {
          constexpr int w = t * WPS + (o - NJ - PPS);
          if constexpr (w < NFW * NS) load_w(NXT{}, w % NFW, w / NFW, c + 1);  // in the order the K-steps use them
        }
      };
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFW, f = m % NFW;
        acc[f][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wreg[PAR][f][t], xf[cur][j], acc[f][j], 0, 0, 0, 0, 0, 0);
        if constexpr (t == NS - 1 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 2) and written its share of
          // the next one (steps 0..2)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<(m * NOPS) / NM, ((m + 1) * NOPS) / NM>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  auto run = [&](auto nj_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int NP = 2 * NJ;
    // Prologue: stage 0 without overlap; the loads left in flight (activations, then weights, of stage 1) are
    // issued in the order the steady state leaves them in at the top of a stage.
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NFW * NS>([&](auto wc) __attribute__((always_inline)) { load_w(S0, decltype(wc)::value % NFW, decltype(wc)::value / NFW, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NP>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NFW * NS>([&](auto wc) __attribute__((always_inline)) { load_w(S1, decltype(wc)::value % NFW, decltype(wc)::value / NFW, 1); });
    __builtin_amdgcn_sched_barrier(0);
    // the claim issued when the tile started has had the prologue's loads to travel behind
    if (claim_now && pass_off == 0 && tid == 0) next_tile_s[tile_par ^ 1] = claimer.resolve();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { read_xf(0, 0, decltype(jc)::value, xf[0]); });
    __builtin_amdgcn_sched_barrier(0);
    int c = 0;
    for (; c + 1 < nst; c += 2) {
      stage(nj_c, S0, c);
      stage(nj_c, S1, c + 1);
    }
    if (c < nst) stage(nj_c, S0, c);
  };
  static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
    if (nj == decltype(n_c)::value) run(n_c);
  });
  // (the LDS reads after the last stage's barrier fetch operands of a stage that does not exist and are not
  // used, so the next pass may overwrite the buffers without another barrier)
  gemm_epilogue<FM, 1, MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                         pid_n * BN + BN <= N, 0, lr, h);
  }  // passes
  // next tile
  if (dyn) {
    // written by thread 0 before this tile's first workgroup barrier; the slot is not written again before the
    // first barrier of the tile after the next, which no wave passes before it has read this value
    tile_par ^= 1;
    pid = claim_now ? __builtin_amdgcn_readfirstlane(next_tile_s[tile_par]) : pid_second;
    ++n_tile;
  } else {
    round0 += (int)gridDim.x;
    const int in_round = live - round0 < (int)gridDim.x ? live - round0 : (int)gridDim.x;
    pid = (int)blockIdx.x < in_round ? round0 + xcd_remap(blockIdx.x, in_round) : -1;
  }
  }  // tiles
  if (dyn) claimer.finish();
}

// ------------------------------------------------------------------------------------------------
// MXFP8 activations x MXFP4 weights in the tile-native layout (prefill): scaled MFMA, no conversion anywhere
// ------------------------------------------------------------------------------------------------
// Both operands stay in their storage formats down to the matrix core: v_mfma_scale_f32_32x32x64_f8f6f4 takes the
// packed e2m1 weights (A operand, format fp4), the e4m3 activations (B operand) and one e8m0 scale byte per lane for
// each, and multiplies both block scales in.  A lane of half h supplies 32 consecutive k of its column / row to one
// instruction, which is exactly one MX block, so the tiled weight layout of the bf16-activation kernel serves as
// it is: piece q of a lane holds k in [s*128 + h*64 + q*32, +32) and byte 2h + q of the stage's scale dword is that
// block's scale (the dword is shifted by 16h once per stage, the instruction's op_sel picks byte q).  The
// activation rows (gathered, one byte per element, 128 bytes per row and stage) are staged through LDS with their
// four e8m0 bytes of the stage in the row's pad.  With a 4-bit and an 8-bit operand the instruction does not pair a
// lane's 32 values one to one: the 8-bit lane of half h holds k' = 16h..16h+15 and 32+16h..32+16h+15 of the
// instruction's 64, while its scale byte still covers k' in [32h, 32h+32), so a lane reads 16 bytes of each of the
// step's two MX blocks (measured with a one-hot probe; exact against a float64 model with random data and scales).
// A K-stage is two MFMA steps (q = 0, 1); structure as in the FP8 kernel: four waves, each owning NFW column
// fragments whose weights go global memory -> register double buffer -> MFMA, all sharing the row fragments of the
// tile through an LDS double buffer; persistent grid, (expert, column tile, row block) tile order.
//
// MXOUT: the output is MX-quantised along N from the fp32 accumulators (after bias, activation and gate weight):
// blocks of 32 output columns, one e8m0 scale byte per block (round-up rule) to y_mx_scale, e4m3 values to y.  A
// wave's 64 accumulator columns are one block with swiglu (two without), half of it in each lane half.
template <int MFW, int NFW, bool SWIGLU>
__device__ __forceinline__ void mx_out_epilogue(const GemmParams& p, f32x16_t (&acc)[NFW][MFW], int expert, int off_m, int start_m, int eM,
                                                int ncol0, int lr, int h) {
  const int N = p.N;
  const int NOUT = SWIGLU ? N / 2 : N;
  const float nalpha_log2e = -p.alpha * 1.4426950408889634f;
  const float limit = p.has_limit ? p.limit : INFINITY;
  uint8_t* yb = reinterpret_cast<uint8_t*>(p.y);
  // everything rows and columns need from memory is fetched before the arithmetic starts: per-row gate weight and
  // destination (rows past the slice read its last row), per-column bias (4 consecutive columns per register group)
  float gam[MFW];
  int64_t dst[MFW];
  bool ok[MFW];
#pragma unroll
  for (int j = 0; j < MFW; ++j) {
    const int row = off_m + j * 32 + lr;  // row inside the slice
    ok[j] = row < eM;
    const int srow = start_m + (ok[j] ? row : eM - 1);
    gam[j] = p.gammas ? load_scalar(p.gammas, srow, p.gammas_is_f32) : 1.0f;
    dst[j] = srow;
    if (p.scatter) {
      const int sr = srow < p.scatter_len ? srow : p.scatter_len - 1;
      const int v = p.scatter[sr];
      dst[j] = srow < p.scatter_len ? v : -1;
    }
  }
  float b4[NFW][4][4];  // [fragment][register group q][i]: bias of column ncol0 + f*32 + 8q + 4h + i
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n0 = ncol0 + f * 32 + 8 * q + 4 * h;
      const int64_t bo = (int64_t)expert * p.bias_stride_e + n0;
      if (!p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) b4[f][q][i] = 0.f;
      } else if (n0 + 4 <= N && p.bias_vec) {
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
  for (int j = 0; j < MFW; ++j) {
    const bool okj = ok[j] && dst[j] >= 0;
    const float g = gam[j];
    // values of this lane: o[f][u][i]; with swiglu 4 outputs per (f, u) at output column (ncol0 + f*32 + 16u + 8h)/2 + i,
    // without 8 outputs at column ncol0 + f*32 + 16u + 8h + i
    constexpr int VO = SWIGLU ? 4 : 8;
    float o[NFW][2][VO];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // registers 8u..8u+3 hold columns 16u + 4h + i, registers 8u+4..8u+7 columns 16u + 8 + 4h + i; after the two
          // lane halves exchange their 4-column groups a lane holds 8 consecutive columns from 16u + 8h
          const float a_lo = acc[f][j][8 * u + i] + b4[f][2 * u][i], a_hi = acc[f][j][8 * u + 4 + i] + b4[f][2 * u + 1][i];
          auto sw = __builtin_amdgcn_permlane32_swap(f32_bits(a_lo), f32_bits(a_hi), false, false);
          v[i] = bits_f32(sw[0]);
          v[4 + i] = bits_f32(sw[1]);
        }
#pragma unroll
        for (int i = 0; i < VO; ++i) o[f][u][i] = SWIGLU ? swiglu_f(v[2 * i], v[2 * i + 1], nalpha_log2e, limit) * g : v[i] * g;
      }
    // MX blocks of 32 output columns: with swiglu the wave's 32 outputs of a row (both fragments, both lane halves),
    // without it one block per fragment.  Columns past the end count as zero.
    constexpr int NB = SWIGLU ? 1 : NFW;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float m = 0.f;
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < VO; ++i) {
            const int col = SWIGLU ? (ncol0 + f * 32 + 16 * u + 8 * h) / 2 + i : ncol0 + f * 32 + 16 * u + 8 * h + i;
            const float a = col < NOUT ? fabsf(o[f][u][i]) : 0.f;
            m = a > m ? a : m;  // (a NaN never wins: the block's scale then comes from its finite values)
          }
      }
      const float other = __shfl_xor(m, 32);
      m = other > m ? other : m;
      const uint32_t sbits = mx_scale_bits(m, TK_E4M3, TK_MX_ROUND_UP);
      const float inv = mx_inv_scale(sbits);
      const int blk_col0 = SWIGLU ? ncol0 / 2 : ncol0 + b * 32;  // first output column of the block
      if (okj && h == 0 && blk_col0 < NOUT) p.y_mx_scale[dst[j] * p.ys_stride_m + blk_col0 / 32] = (uint8_t)(sbits >> 23);
#pragma unroll
      for (int f = 0; f < NFW; ++f) {
        if (!SWIGLU && f != b) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int col0 = SWIGLU ? (ncol0 + f * 32 + 16 * u + 8 * h) / 2 : ncol0 + f * 32 + 16 * u + 8 * h;
          float qv[VO];
#pragma unroll
          for (int i = 0; i < VO; ++i) qv[i] = mx_clamp(o[f][u][i] * inv, 448.0f);
          uint8_t* yrow = yb + dst[j] * p.y_stride_m + col0;
          if (okj && col0 + VO <= NOUT && p.y_vec) {
            int w0 = 0;
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], w0, false);
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], w0, true);
            if constexpr (VO == 8) {
              int w1 = 0;
              w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], w1, false);
              w1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], w1, true);
              *reinterpret_cast<uint2*>(yrow) = make_uint2((uint32_t)w0, (uint32_t)w1);
            } else {
              *reinterpret_cast<uint32_t*>(yrow) = (uint32_t)w0;
            }
          } else if (okj) {
#pragma unroll
            for (int i = 0; i < VO; ++i)
              if (col0 + i < NOUT) yrow[i] = (uint8_t)e4m3_byte(qv[i]);
          }
        }
      }
    }
  }
}

template <int BLKM, int MFW, int NFW, bool SWIGLU, bool MXOUT>
__global__ __launch_bounds__(256) void moe_gemm_mx8n_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, BM = MFW * 32, BN = 128 * NFW, KC = 128, NS = 2;
  constexpr int XPITCH = KC + 16;  // 128 value bytes, 4 scale bytes, pad
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = BM / 32;  // 16-byte activation pieces per thread per stage (8 pieces per row, 32 rows per sweep)
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);  // column quarter of the tile
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;  // stages of 128
  const int grid = (int)gridDim.x;
  const int live = p.slice_sizes ? p.block_offs[p.n_slices] * p.grid_n : p.total_tiles;
  for (int round0 = 0; round0 < live; round0 += grid) {
  const int in_round = live - round0 < grid ? live - round0 : grid;
  if ((int)blockIdx.x >= in_round) break;
  const int pid = round0 + xcd_remap(blockIdx.x, in_round);
  int expert, blk_off, start_m, eM, pid_n;
  if (p.slice_sizes) {
    expert = p.block_sched[pid / p.grid_n] & 0xFFFF;
    const int first = p.block_offs[expert];
    const int nb = p.block_offs[expert + 1] - first;
    const int local = pid - first * p.grid_n;
    pid_n = local / nb;
    blk_off = (local - pid_n * nb) * BLKM;
    start_m = p.slice_offs[expert];
    eM = p.slice_sizes[expert];
  } else {
    pid_n = pid % p.grid_n;
    expert = 0;
    blk_off = (pid / p.grid_n) * BLKM;
    start_m = 0;
    eM = p.M;
  }
  const int blk_rows = (eM - blk_off) < BLKM ? (eM - blk_off) : BLKM;
  for (int pass_off = 0; pass_off < blk_rows; pass_off += BM) {
  const int off_m = blk_off + pass_off;
  const int rows = (blk_rows - pass_off) < BM ? (blk_rows - pass_off) : BM;
  const int nj = (rows + FM - 1) / FM;  // row fragments that hold valid rows (1..MFW)

  // ---- activation staging: piece j of this thread = row 32 j + tid/8, 16-byte chunk tid%8 of the stage; the
  // stage's four scale bytes of row `tid` (tid < BM) travel with them ----
  const int xc = tid & 7;
  const uint8_t* xptr[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int row = off_m + (tid >> 3) + 32 * j;
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xptr[j] = p.x + src * p.x_stride_m;
  }
  const uint8_t* xsptr;
  {
    int row = off_m + (tid < BM ? tid : BM - 1);
    row = row < eM ? row : eM - 1;
    const int64_t src = p.gather ? (int64_t)p.gather[start_m + row] : (int64_t)(start_m + row);
    xsptr = p.x_mx_scale + src * p.xs_stride_m;
  }
  const int xlds0 = (tid >> 3) * XPITCH + xc * 16;  // piece j at xlds0 + j*32*XPITCH
  const int kblocks = (K + 31) >> 5;                // scale bytes per activation row (>= 4, checked by the host)

  const int nfr = (N + 31) >> 5;
  const uint8_t* wptr[NFW];
  const uint8_t* sptr[NFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f) {
    int F = pid_n * (BN / 32) + nw * NFW + f;
    F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
    wptr[f] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F * nst * 2048 + lane * 16;
    sptr[f] = p.w_scale + (int64_t)expert * p.ws_stride_e + (int64_t)F * nst * 128 + lr * 4;
  }

  typename FR::acc_t acc[NFW][MFW];
#pragma unroll
  for (int f = 0; f < NFW; ++f)
#pragma unroll
    for (int j = 0; j < MFW; ++j)
#pragma unroll
      for (int i = 0; i < FR::NACC; ++i) acc[f][j][i] = 0.f;

  // Register rings: a stage of two MFMA steps is too short to cover a memory round trip, so the weights of stage c + 3
  // and the activations of stage c + 3 are requested while stage c computes (weights: four slots, stage c uses slot
  // c % 4; activations: two slots, slot (c + 1) % 2 holds stage c + 1 until stage c has written it to LDS).
  constexpr int WD = 4, XD = 2;
  u32x4_t xreg[XD][XCH];
  uint32_t xsreg[XD] = {0, 0};
  int xsshift[XD] = {0, 0};   // blocks by which the dword in xsreg starts before block 4 s of its stage
  u32x4_t wraw[WD][NFW][NS];  // [ring slot][column fragment][step]
  uint32_t sd[WD][NFW];       // the stage's four weight scale bytes of this lane's column
  i32x8_t xf[2][MFW];         // [step parity][row fragment]
  uint32_t xs[2][MFW];        // [stage parity]: the stage's activation scale bytes of this lane's rows, this half's two in bytes 0 / 1

  // Loads are unconditional: rows past the last valid row re-read it, k past K re-reads the row's last 16 bytes /
  // last scale bytes (the padded weights there are zero), stages past the last one re-read the last stage.
  auto load_x_piece = [&](int j, int s, int slot) __attribute__((always_inline)) {
    int k0 = s * KC + xc * 16;
    k0 = k0 < K - 16 ? k0 : K - 16;
    xreg[slot][j] = *reinterpret_cast<const u32x4_t*>(xptr[j] + k0);
  };
  auto load_x_scale = [&](int s, int slot) __attribute__((always_inline)) {
    // four scale bytes from block 4 s on (any alignment); a stage that reaches past the row's last block reads the
    // last four blocks instead.  Only the load is issued here: the bytes are moved into place when they go to LDS
    // (anything computed from the loaded value now would make the wave wait for it on the spot).
    int b0 = s * 4;
    b0 = b0 < kblocks - 4 ? b0 : kblocks - 4;
    uint32_t v;
    __builtin_memcpy(&v, xsptr + b0, 4);
    xsreg[slot] = v;
    xsshift[slot] = s * 4 - b0;
  };
  auto store_x_piece = [&](int j, int buf, int slot) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 32 * XPITCH) = xreg[slot][j];
  };
  auto store_x_scale = [&](int buf, int slot) __attribute__((always_inline)) {
    // block 4 s of the stage goes to byte 0; blocks past the row's end get the neutral scale 2^0 (their weights are zero)
    const int sh = xsshift[slot] < 4 ? xsshift[slot] : 4;
    const uint64_t wide = ((uint64_t)0x7F7F7F7Fu << 32) | xsreg[slot];
    const uint32_t v = (uint32_t)(wide >> (8 * sh));
    if (tid < BM) *reinterpret_cast<uint32_t*>(lds + buf * XBYTES + tid * XPITCH + KC) = v;
  };
  auto load_w = [&](auto slot_c, int s) __attribute__((always_inline)) {
    constexpr int SL = decltype(slot_c)::value;
    s = s < nst ? s : nst - 1;
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      wraw[SL][f][0] = *reinterpret_cast<const u32x4_t*>(wptr[f] + (int64_t)s * 2048);
      wraw[SL][f][1] = *reinterpret_cast<const u32x4_t*>(wptr[f] + (int64_t)s * 2048 + 1024);
      sd[SL][f] = *reinterpret_cast<const uint32_t*>(sptr[f] + (int64_t)s * 128);
    }
  };
  auto read_xf = [&](int buf, int q, int j, i32x8_t (&out)[MFW]) __attribute__((always_inline)) {
    // (the instruction pairs the fp4 operand's nibble i of lane half hh with the 8-bit operand's k = 32 hh + i, which
    // it takes from byte i of half 0 for i < 16 and byte i - 16 of half 1 otherwise, and likewise bytes 16..31 for the
    // second 32: a lane of half h therefore supplies bytes [16 h, 16 h + 16) of both of the step's MX blocks)
    const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + q * 32 + h * 16;
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 64);
    out[j] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_xs = [&](int buf, int j, uint32_t (&out)[MFW]) __attribute__((always_inline)) {
    out[j] = *reinterpret_cast<const uint32_t*>(lds + buf * XBYTES + (j * FM + lr) * XPITCH + KC) >> (16 * h);
  };

  template_int<0> S0;
  template_int<1> S1;
  template_int<2> S2;
  template_int<3> S3;

  // One stage.  NJ = row fragments with valid rows; WS4 = c % 4: weight ring slot, its low bit the LDS buffer and the
  // activation scale set.  The MFMAs of step q are interleaved with the LDS reads of the next step's activation
  // fragments (during step 1: the next stage's step 0 and its scale bytes, behind the barrier), and during step 0
  // with the staging of the next stage's activations, the refill of their registers and the weight loads.
  auto stage = [&](auto nj_c, auto ws_c, int c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    constexpr int WS4 = decltype(ws_c)::value;
    constexpr int PAR = WS4 & 1;
    using WSL = template_int<(WS4 + WD - 1) % WD>;  // slot to refill with stage c + WD - 1 (stage c - 1 used it)
    constexpr int XS = (WS4 + 1) % XD;              // activation register slot holding stage c + 1
    constexpr int NM = NJ * NFW;
    constexpr int NOPS = 2 * NJ + 2;  // NJ reads, NJ staging pieces, the scale staging, the weight loads
    uint32_t sdh[NFW];
#pragma unroll
    for (int f = 0; f < NFW; ++f) sdh[f] = sd[WS4][f] >> (16 * h);
    static_for<0, NS>([&](auto q_c) __attribute__((always_inline)) {
      constexpr int q = decltype(q_c)::value;
      constexpr int cur = q & 1, nxt = cur ^ 1;
      auto op = [&](auto o_c) __attribute__((always_inline)) {
        constexpr int o = decltype(o_c)::value;
        if constexpr (o < NJ) {
          if constexpr (q == 0) {
            read_xf(PAR, 1, o, xf[nxt]);
          } else {
            read_xf(PAR ^ 1, 0, o, xf[nxt]);
            read_xs(PAR ^ 1, o, xs[PAR ^ 1]);
          }
        } else if constexpr (o < 2 * NJ) {
          if constexpr (q == 0) {
            constexpr int j = o - NJ;
            store_x_piece(j, PAR ^ 1, XS);
            load_x_piece(j, c + 1 + XD, XS);
          }
        } else if constexpr (o == 2 * NJ) {
          if constexpr (q == 0) {
            store_x_scale(PAR ^ 1, XS);
            load_x_scale(c + 1 + XD, XS);
          }
        } else {
          if constexpr (q == 0) load_w(WSL{}, c + WD - 1);
        }
      };
      static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int j = m / NFW, f = m % NFW;
        const u32x4_t wv = wraw[WS4][f][q];
        const i32x8_t a = {(int)wv.x, (int)wv.y, (int)wv.z, (int)wv.w, 0, 0, 0, 0};
        acc[f][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, xf[cur][j], acc[f][j], 4 /* A: e2m1 */, 0 /* B: e4m3 */, q, (int)sdh[f], q,
                                                                     (int)xs[PAR][j]);
        if constexpr (q == NS - 1 && m == 0) {
          // every wave has fetched its last operands of this buffer (during step 0) and written its share of the
          // next one (step 0)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        static_for<(m * NOPS) / NM, ((m + 1) * NOPS) / NM>(op);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  auto run = [&](auto nj_c) __attribute__((always_inline)) {
    constexpr int NJ = decltype(nj_c)::value;
    // Prologue: stage 0 without overlap; the loads left in flight (activations, scales, weights of stage 1, then of
    // stage 2) are issued in the order the steady state leaves them in at the top of a stage.
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0, 0); });
    load_x_scale(0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S0, 0);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0, 0); });
    store_x_scale(0, 0);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1, 1); });
    load_x_scale(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S1, 1);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 2, 0); });
    load_x_scale(2, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(S2, 2);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) {
      read_xf(0, 0, decltype(jc)::value, xf[0]);
      read_xs(0, decltype(jc)::value, xs[0]);
    });
    __builtin_amdgcn_sched_barrier(0);
    // all stages of a group always run inside the loop (a path that skips some and returns to the loop header would
    // make the header's wait counts cover the loads just issued)
    int c = 0;
    for (; c + 3 < nst; c += 4) {
      stage(nj_c, S0, c);
      stage(nj_c, S1, c + 1);
      stage(nj_c, S2, c + 2);
      stage(nj_c, S3, c + 3);
    }
    if (c < nst) stage(nj_c, S0, c);
    if (c + 1 < nst) stage(nj_c, S1, c + 1);
    if (c + 2 < nst) stage(nj_c, S2, c + 2);
  };
  static_for<1, MFW + 1>([&](auto n_c) __attribute__((always_inline)) {
    if (nj == decltype(n_c)::value) run(n_c);
  });
  // (the LDS reads after the last stage's barrier fetch operands of a stage that does not exist and are not
  // used, so the next pass may overwrite the buffers without another barrier)
  if constexpr (MXOUT)
    mx_out_epilogue<MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM, lr, h);
  else
    gemm_epilogue<FM, 1, MFW, NFW, SWIGLU>(p, acc, expert, off_m, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                           pid_n * BN + BN <= N, 0, lr, h);
  }  // passes
  }  // rounds
}

template <int MR, int NFD>
int32_t launch_mxd_n(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  GemmParams q = p;
  q.total_tiles = grid_m;  // row blocks in the non-ragged case
  // sized for a K-split of 4 (one fragment group per workgroup); with a smaller split the surplus leaves at once
  const int64_t grid = (int64_t)grid_m * ((cdiv(cdiv(p.N, 32), NFD) + 7) & ~int64_t(7));
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  if (swiglu)
    hipLaunchKernelGGL((moe_gemm_mxd_kernel<MR, NFD, true>), dim3((unsigned)grid), dim3(256), 0, st, q);
  else
    hipLaunchKernelGGL((moe_gemm_mxd_kernel<MR, NFD, false>), dim3((unsigned)grid), dim3(256), 0, st, q);
  return check_launch("moe_gemm_mxd_kernel");
}
template <int MR>
int32_t launch_mxd(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  // Two fragments per wave halve the activation reads (which come from L2) at the price of half as many waves.  With
  // few rows only a few experts are live and the kernel needs every wave it can get to keep HBM busy; from about a
  // hundred rows on the activation traffic is what limits it.  (Measured at 128 experts, top-4: 16 tokens are 6 %
  // faster with one fragment, 64 tokens 8 % faster with two.)
  return p.M >= 128 ? launch_mxd_n<MR, 2>(p, grid_m, swiglu, st) : launch_mxd_n<MR, 1>(p, grid_m, swiglu, st);
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

template <int BLKM, int MFW, int NFW, int G, int WD, int XD>
int32_t launch_mxn(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * G * (128 * 2 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  // persistent grid: one workgroup per CU (a wave's registers leave no room for a second one on its SIMD)
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256 * G), LDS_BYTES, st, q);
    return check_launch("moe_gemm_mxn_kernel");
  };
  if (swiglu) return launch(moe_gemm_mxn_kernel<BLKM, MFW, NFW, G, WD, XD, true>);
  return launch(moe_gemm_mxn_kernel<BLKM, MFW, NFW, G, WD, XD, false>);
}

template <int BLKM, int MFW, int NFW>
int32_t launch_f8n(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * (256 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  // persistent grid, one workgroup per CU (the register ring and the accumulators take a wave's whole budget)
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS_BYTES, st, q);
    return check_launch("moe_gemm_f8n_kernel");
  };
  if (swiglu) return launch(moe_gemm_f8n_kernel<BLKM, MFW, NFW, true>);
  return launch(moe_gemm_f8n_kernel<BLKM, MFW, NFW, false>);
}

template <int BLKM, int MFW, int NFW>
int32_t launch_mx8n(const GemmParams& p, int grid_m, bool swiglu, bool mxout, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * MFW * 32 * (128 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 128 * NFW);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);  // persistent grid, one workgroup per CU
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS_BYTES, st, q);
    return check_launch("moe_gemm_mx8n_kernel");
  };
  if (swiglu && mxout) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, true, true>);
  if (swiglu) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, true, false>);
  if (mxout) return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, false, true>);
  return launch(moe_gemm_mx8n_kernel<BLKM, MFW, NFW, false, false>);
}

template <int WK, int FM, int WM, int WN, int MFW, int NFW, int KS>
int32_t launch_cfg(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int BM = WM * MFW * FM;
  constexpr int BN = WN * NFW * FM;
  constexpr int KC = 128 * KS;
  constexpr int WROW = WK == WK_MXFP4 ? KC / 2 : (WK == WK_FP8 ? KC : KC * 2);
  constexpr int LDS_BYTES = 2 * (BM * (KC * 2 + 16) + BN * (WROW + 16));
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, BN);
  const int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), LDS_BYTES, st, q);
    return check_launch("moe_gemm_kernel");
  };
  if (swiglu) return launch(moe_gemm_kernel<WK, FM, WM, WN, MFW, NFW, KS, true>);
  return launch(moe_gemm_kernel<WK, FM, WM, WN, MFW, NFW, KS, false>);
}

template <int WK>
int32_t launch_wk(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  //                      FM  WM WN MFW NFW KS
  if constexpr (WK == WK_MXFP4) {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 2>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 2>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 4, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 4, 1>(p, grid_m, swiglu, st);
    }
  } else if constexpr (WK == WK_FP8) {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 2>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 2>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 4, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 4, 1>(p, grid_m, swiglu, st);
    }
  } else {
    switch (block_m) {
      case 16:
        return launch_cfg<WK, 16, 1, 4, 1, 2, 1>(p, grid_m, swiglu, st);
      case 32:
        return launch_cfg<WK, 16, 1, 4, 2, 2, 1>(p, grid_m, swiglu, st);
      case 64:
        return launch_cfg<WK, 32, 2, 2, 1, 2, 1>(p, grid_m, swiglu, st);
      case 128:
        return launch_cfg<WK, 32, 2, 2, 2, 2, 1>(p, grid_m, swiglu, st);
    }
  }
  return fail(TK_ERR_INVALID, "tk_moe_gemm: block_m must be 16, 32, 64 or 128 (got %d)", block_m);
}

}  // namespace
}  // namespace tk

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
  const bool mx_out = d->y_dtype == TK_E4M3 && d->y_mx_scale != nullptr;
  if (d->y_dtype != TK_BF16 && !f16 && !(mx_out && mx_act)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: output must be bf16, or e4m3 with y_mx_scale on the MXFP8-activation path (dtype %d)", d->y_dtype);
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
    if (!(d->w_layout == TK_W_TILED && d->w_dtype == TK_E2M1 && (d->block_m == 16 || d->block_m == 32)))
      return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the fused top-k combine needs tiled MXFP4 weights and block_m 16 or 32");
    if (!d->scatter_indx || !d->combine_out || !d->combine_counters || d->activation != TK_ACT_NONE)
      return fail(TK_ERR_INVALID, "tk_moe_gemm: the fused top-k combine needs scatter_indx, combine_out and combine_counters, and no activation");
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
  p.x_mx_scale = static_cast<const uint8_t*>(d->x_mx_scale);
  p.xs_stride_m = d->xs_stride_m;
  p.y_mx_scale = static_cast<uint8_t*>(d->y_mx_scale);
  p.ys_stride_m = d->ys_stride_m;
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
    //                                          BLKM MFW NFW
    if (d->block_m == 256) return launch_f8n<256, 4, 2>(p, d->grid_m, swiglu, st);
    return launch_f8n<128, 4, 2>(p, d->grid_m, swiglu, st);
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
    if (mx_out) {
      const int64_t n_out = swiglu ? d->N / 2 : d->N;
      if (n_out % 32) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: an MX-quantised output needs N_out %% 32 == 0 (got %lld)", (long long)n_out);
      p.y_vec = (d->y_stride_m % 8 == 0) && ((reinterpret_cast<uintptr_t>(d->y) & 7) == 0);
    }
    p.w_stride_e = d->w_stride_e;
    p.w_nst = (int32_t)nst;
    //                                       BLKM MFW NFW
    if (d->block_m == 256) return launch_mx8n<256, 5, 2>(p, d->grid_m, swiglu, mx_out, st);
    return launch_mx8n<128, 4, 2>(p, d->grid_m, swiglu, mx_out, st);
  }
  if (d->w_layout == TK_W_TILED) {
    if (d->w_dtype != TK_E2M1 || !d->w_mx_scale || d->x_dtype != TK_BF16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: the tiled weight layout holds MXFP4 weights for bf16 activations");
    if (d->block_m != 16 && d->block_m != 32 && d->block_m != 64 && d->block_m != 128 && d->block_m != 256) return fail(TK_ERR_INVALID, "tk_moe_gemm: block_m must be 16, 32, 64, 128 or 256 (got %d)", d->block_m);
    if (d->block_m >= 64) {
      // the prefill kernels address activation rows with 32-bit byte offsets from x
      const int64_t rows = d->x_rows > 0 ? d->x_rows : (d->gather_indx ? 0 : d->M);
      if (d->x_stride_m * 2 >= (int64_t)1 << 32 || rows * d->x_stride_m * 2 > (int64_t)1 << 32)
        return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: activations of 4 GiB and more are not supported with tiled MXFP4 weights (%lld rows, row stride %lld)", (long long)rows, (long long)d->x_stride_m);
    }
    if (d->block_m >= 64) {
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
    //                                  BLKM MFW NFW G WD XD
    if (d->block_m == 16) return launch_mxd<1>(p, d->grid_m, swiglu, st);
    if (d->block_m == 32) return launch_mxd<2>(p, d->grid_m, swiglu, st);
    if (d->block_m == 64) return launch_mxn<64, 2, 2, 1, 4, 2>(p, d->grid_m, swiglu, st);
    if (d->block_m == 256) return launch_mxn<256, 5, 2, 1, 2, 1>(p, d->grid_m, swiglu, st);
    return launch_mxn<128, 4, 2, 1, 4, 2>(p, d->grid_m, swiglu, st);
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
    return launch_wk<WK_MXFP4>(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_BF16) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with bf16 weights");
    if (d->w_stride_n % 8 || d->w_stride_e % 8 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e * 2;
    p.w_stride_n = d->w_stride_n * 2;
    return launch_wk<WK_BF16>(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_F16) {
    // fp16 x fp16 -> fp16 (v_mfma_f32_*_f16); same data path as bf16
    if (d->x_dtype != TK_F16 || d->y_dtype != TK_F16) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: fp16 weights go with fp16 activations and an fp16 output");
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with fp16 weights");
    if (d->w_stride_n % 8 || d->w_stride_e % 8 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e * 2;
    p.w_stride_n = d->w_stride_n * 2;
    return launch_wk<WK_F16>(p, d->block_m, d->grid_m, swiglu, st);
  }
  if (d->w_dtype == TK_E4M3) {
    if (d->w_mx_scale) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: MX scales with e4m3 weights");
    if (d->w_stride_n % 16 || d->w_stride_e % 16 || (reinterpret_cast<uintptr_t>(d->w) & 15)) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight columns must be 16-byte aligned");
    p.w_stride_e = d->w_stride_e;
    p.w_stride_n = d->w_stride_n;
    return launch_wk<WK_FP8>(p, d->block_m, d->grid_m, swiglu, st);
  }
  return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: weight dtype %d is not supported", d->w_dtype);
}
