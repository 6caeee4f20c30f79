// MX quantise / dequantise kernels for gfx950 (HBM-bound byte work).
//
// Source layouts handled without a transposed temporary:
//   rows : the quantised axis is the unit-stride one; 4 lanes share a block of 32, each holds 8
//          consecutive elements, the block maximum is a 2-step lane exchange.
//   cols : the quantised axis is strided and the INNER axis is unit-stride (a weight [E, K, N]
//          quantised along K); a lane owns one or two columns and walks 32 rows, so every load of a
//          wave is one contiguous row segment and the 32-element reduction is register-local.
//   tile : the cols case for 16-bit tensors, with an LDS transpose so that the quantised bytes of a column move
//          as full 128-byte lines (mx_down_tile / mx_up_tile).
#include "mx_math.h"

namespace tk {
namespace {

constexpr int kThreads = 256;

template <int DT>
struct Elem;
template <>
struct Elem<TK_F32> {
  typedef float T;
  static __device__ float load(const T* p) { return *p; }
  static __device__ void store(T* p, float v) { *p = v; }
  static __device__ float max_finite() { return 3.4028234663852886e+38f; }
};
template <>
struct Elem<TK_BF16> {
  typedef uint16_t T;
  static __device__ float load(const T* p) { return bf16_bits_to_f32(*p); }
  static __device__ void store(T* p, float v) { *p = f32_to_bf16_bits(v); }
  static __device__ float max_finite() { return 3.3895313892515355e+38f; }
};
template <>
struct Elem<TK_F16> {
  typedef uint16_t T;
  static __device__ float load(const T* p) { return f16_bits_to_f32(*p); }
  static __device__ void store(T* p, float v) { *p = f32_to_f16_bits(v); }
  static __device__ float max_finite() { return 65504.0f; }
};

// Index of the output line (run of one (outer, inner) coordinate along the quantised axis).  The inner
// extent is mid x last with `last` fastest in the source; outputs order lines (outer, last, mid), which
// is the order `x.transpose(axis, -1)` gives them.
__device__ inline int64_t line_of(int64_t o, int64_t col, int64_t inner, int64_t inner_last) {
  if (inner_last == inner) return o * inner + col;
  const int64_t m = col / inner_last;
  const int64_t l = col - m * inner_last;
  return (o * inner_last + l) * (inner / inner_last) + m;
}

template <int KIND>
__device__ inline uint32_t quant_byte(float q) {
  if (KIND == TK_E4M3) return e4m3_byte(mx_clamp(q, 448.0f));
  return e5m2_byte(mx_clamp(q, 57344.0f));
}

template <int KIND>
__device__ inline float elem_f32(uint32_t b) {
  if (KIND == TK_E4M3) return e4m3_to_f32(b);
  return e5m2_to_f32(b);
}

// ---------------------------------------------------------------------------------------------
// downcast, quantised axis contiguous: src [rows, L] with row stride `ld`
// ---------------------------------------------------------------------------------------------
template <int SRC, int KIND>
__global__ __launch_bounds__(kThreads) void mx_down_rows(const typename Elem<SRC>::T* __restrict__ src, int64_t ld,
                                                         int64_t rows, int64_t L, uint8_t* __restrict__ out_vals,
                                                         uint8_t* __restrict__ out_scales, int rounding) {
  const int64_t groups_per_row = L / 8;
  const int64_t total = rows * groups_per_row;
  const int64_t gid = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (gid >= total) return;  // total % 4 == 0, so a quad of lanes is either fully in or fully out
  const int64_t row = gid / groups_per_row;
  const int64_t g = gid - row * groups_per_row;
  const typename Elem<SRC>::T* p = src + row * ld + g * 8;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = Elem<SRC>::load(p + i);
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) m = fmaxf(m, fabsf(v[i]));
  m = fmaxf(m, __shfl_xor(m, 1));
  m = fmaxf(m, __shfl_xor(m, 2));
  const uint32_t sbits = mx_scale_bits(m, KIND, rounding);
  const float inv = mx_inv_scale(sbits);
  if (KIND == TK_E2M1) {
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) packed |= e2m1_code(v[i] * inv) << (4 * i);
    *reinterpret_cast<uint32_t*>(out_vals + row * (L / 2) + g * 4) = packed;
  } else {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) lo |= quant_byte<KIND>(v[i] * inv) << (8 * i);
#pragma unroll
    for (int i = 0; i < 4; ++i) hi |= quant_byte<KIND>(v[4 + i] * inv) << (8 * i);
    *reinterpret_cast<uint2*>(out_vals + row * L + g * 8) = make_uint2(lo, hi);
  }
  if ((g & 3) == 0) out_scales[row * (L / 32) + (g >> 2)] = (uint8_t)(sbits >> 23);
}

// ---------------------------------------------------------------------------------------------
// downcast, inner axis contiguous: src [outer, L, inner], stride_inner == 1
// tile = 4 blocks of 32 rows x (64*CPT) columns per 256-thread workgroup; wave w owns block w
// ---------------------------------------------------------------------------------------------
template <int SRC, int KIND, int CPT>
__global__ __launch_bounds__(kThreads) void mx_down_cols(const typename Elem<SRC>::T* __restrict__ src,
                                                         int64_t stride_outer, int64_t stride_axis, int64_t L,
                                                         int64_t inner, int64_t inner_last, int64_t col_tiles,
                                                         int64_t blk_tiles, uint8_t* __restrict__ out_vals,
                                                         uint8_t* __restrict__ out_scales, int rounding) {
  typedef typename Elem<SRC>::T T;
  int64_t bid = blockIdx.x;
  const int64_t ct = bid % col_tiles;
  bid /= col_tiles;
  const int64_t bt = bid % blk_tiles;
  const int64_t o = bid / blk_tiles;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t blk = bt * 4 + wave;
  const int64_t col = (ct * 64 + lane) * CPT;
  if (blk >= L / 32 || col >= inner) return;
  const T* p = src + o * stride_outer + blk * 32 * stride_axis + col;
  float v[32][CPT];
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    if (CPT == 2) {
      if (sizeof(T) == 2) {
        uint32_t w = *reinterpret_cast<const uint32_t*>(p + i * stride_axis);
        uint16_t a = (uint16_t)(w & 0xFFFFu), b = (uint16_t)(w >> 16);
        v[i][0] = Elem<SRC>::load(reinterpret_cast<const T*>(&a));
        v[i][CPT - 1] = Elem<SRC>::load(reinterpret_cast<const T*>(&b));
      } else {
        float2 w = *reinterpret_cast<const float2*>(p + i * stride_axis);
        v[i][0] = w.x;
        v[i][CPT - 1] = w.y;
      }
    } else {
      v[i][0] = Elem<SRC>::load(p + i * stride_axis);
    }
  }
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) m = fmaxf(m, fabsf(v[i][c]));
    const uint32_t sbits = mx_scale_bits(m, KIND, rounding);
    const float inv = mx_inv_scale(sbits);
    const int64_t line = line_of(o, col + c, inner, inner_last);
    if (KIND == TK_E2M1) {
      uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 32; ++i) w[i >> 3] |= e2m1_code(v[i][c] * inv) << (4 * (i & 7));
      *reinterpret_cast<uint4*>(out_vals + line * (L / 2) + blk * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 32; ++i) w[i >> 2] |= quant_byte<KIND>(v[i][c] * inv) << (8 * (i & 3));
      uint4* dst = reinterpret_cast<uint4*>(out_vals + line * L + blk * 32);
      dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
      dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
    }
    out_scales[line * (L / 32) + blk] = (uint8_t)(sbits >> 23);
  }
}

// ---------------------------------------------------------------------------------------------
// upcast, quantised axis contiguous in the output: out [rows, L] with row stride `ld`
// ---------------------------------------------------------------------------------------------
template <int KIND, int DST>
__global__ __launch_bounds__(kThreads) void mx_up_rows(const uint8_t* __restrict__ vals,
                                                       const uint8_t* __restrict__ scales, int64_t rows, int64_t L,
                                                       typename Elem<DST>::T* __restrict__ out, int64_t ld) {
  const int64_t groups_per_row = L / 8;
  const int64_t total = rows * groups_per_row;
  const int64_t gid = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (gid >= total) return;
  const int64_t row = gid / groups_per_row;
  const int64_t g = gid - row * groups_per_row;
  const uint32_t sb = scales[row * (L / 32) + (g >> 2)];
  const float mf = Elem<DST>::max_finite();
  float v[8];
  if (KIND == TK_E2M1) {
    const uint32_t packed = *reinterpret_cast<const uint32_t*>(vals + row * (L / 2) + g * 4);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      v[i] = mx_dequant(bf16_bits_to_f32((uint16_t)e2m1_to_bf16_bits((packed >> (4 * i)) & 0xFu)), sb, mf, false);
  } else {
    const uint2 w = *reinterpret_cast<const uint2*>(vals + row * L + g * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = mx_dequant(elem_f32<KIND>((w.x >> (8 * i)) & 0xFFu), sb, mf, KIND == TK_E5M2);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[4 + i] = mx_dequant(elem_f32<KIND>((w.y >> (8 * i)) & 0xFFu), sb, mf, KIND == TK_E5M2);
  }
  typename Elem<DST>::T* q = out + row * ld + g * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i) Elem<DST>::store(q + i, v[i]);
}

// ---------------------------------------------------------------------------------------------
// upcast, inner axis contiguous in the output: out [outer, L, inner], ostride_inner == 1
// ---------------------------------------------------------------------------------------------
template <int KIND, int DST, int CPT>
__global__ __launch_bounds__(kThreads) void mx_up_cols(const uint8_t* __restrict__ vals,
                                                       const uint8_t* __restrict__ scales, int64_t L, int64_t inner,
                                                       int64_t inner_last, int64_t col_tiles, int64_t blk_tiles,
                                                       typename Elem<DST>::T* __restrict__ out,
                                                       int64_t ostride_outer, int64_t ostride_axis) {
  typedef typename Elem<DST>::T T;
  int64_t bid = blockIdx.x;
  const int64_t ct = bid % col_tiles;
  bid /= col_tiles;
  const int64_t bt = bid % blk_tiles;
  const int64_t o = bid / blk_tiles;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t blk = bt * 4 + wave;
  const int64_t col = (ct * 64 + lane) * CPT;
  if (blk >= L / 32 || col >= inner) return;
  const float mf = Elem<DST>::max_finite();
  float v[32][CPT];
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int64_t line = line_of(o, col + c, inner, inner_last);
    const uint32_t sb = scales[line * (L / 32) + blk];
    if (KIND == TK_E2M1) {
      const uint4 w4 = *reinterpret_cast<const uint4*>(vals + line * (L / 2) + blk * 16);
      const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
      for (int i = 0; i < 32; ++i)
        v[i][c] = mx_dequant(bf16_bits_to_f32((uint16_t)e2m1_to_bf16_bits((w[i >> 3] >> (4 * (i & 7))) & 0xFu)), sb,
                             mf, false);
    } else {
      const uint4* src = reinterpret_cast<const uint4*>(vals + line * L + blk * 32);
      const uint4 a = src[0], b = src[1];
      const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 32; ++i)
        v[i][c] = mx_dequant(elem_f32<KIND>((w[i >> 2] >> (8 * (i & 3))) & 0xFFu), sb, mf, KIND == TK_E5M2);
    }
  }
  T* q = out + o * ostride_outer + blk * 32 * ostride_axis + col;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    if (CPT == 2 && sizeof(T) == 2) {
      uint16_t a, b;
      Elem<DST>::store(reinterpret_cast<T*>(&a), v[i][0]);
      Elem<DST>::store(reinterpret_cast<T*>(&b), v[i][CPT - 1]);
      *reinterpret_cast<uint32_t*>(q + i * ostride_axis) = (uint32_t)a | ((uint32_t)b << 16);
    } else if (CPT == 2) {
      *reinterpret_cast<float2*>(q + i * ostride_axis) = make_float2(v[i][0], v[i][CPT - 1]);
    } else {
      Elem<DST>::store(q + i * ostride_axis, v[i][0]);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// 16-bit sources / destinations with the inner axis contiguous, through an LDS transpose.
// A workgroup takes 256 columns x NB blocks of 32 rows, NB chosen so that the NB blocks of one column are
// 128 output bytes (8 blocks of e2m1, 4 of fp8): the quantised bytes of a column are then moved as one full
// 128-byte line (8 lanes x 16 bytes) instead of 16- or 32-byte pieces of 64 different lines per instruction,
// and a lane walks its rows with 8-byte accesses (4 columns), so a wave covers 512 contiguous bytes per row.
// ---------------------------------------------------------------------------------------------
constexpr int kTileCols = 256;
constexpr int kTilePitch = 128 + 16;  // LDS bytes per column
// LDS row of tile column c: a lane's four adjacent columns are spread 65 rows apart, so the 16-byte accesses of
// consecutive lanes (columns c, c + 4, ...) fall 144 bytes apart and take different banks
constexpr int kTileRows = 64 + 65 * 3;
__device__ __forceinline__ int tile_row(int c) { return (c >> 2) + 65 * (c & 3); }

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Tiles are renumbered so that consecutive
// tiles run on ONE XCD at about the same time, and the tiles of one column range are numbered consecutively along
// the quantised axis: a column's quantised bytes (1440 per 2880 values of e2m1) are not a multiple of the 128-byte
// line, so neighbouring tiles share the lines at their seams and the 64-byte pieces of the scale rows; in one L2
// those are fetched (or written back) once, in two L2s twice.
__device__ __forceinline__ int64_t tile_order(int64_t pid, int64_t total) {
  const int64_t per = total / 8, extra = total % 8;
  const int64_t grp = pid % 8, local = pid / 8;
  return grp * per + (grp < extra ? grp : extra) + local;
}

typedef __attribute__((ext_vector_type(2))) unsigned short u16x2_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}
// two 16-bit floats (low half first) / scale -> two e2m1 codes in byte `SEL` of `old` (first value in the low nibble)
template <int SRC>
__device__ __forceinline__ uint32_t cvt_pk_fp4(uint32_t old, uint32_t pair, float scale, int sel) {
  if constexpr (SRC == TK_BF16) {
    const bf16x2_t v = __builtin_bit_cast(bf16x2_t, pair);
    return sel == 0   ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, v, scale, 0)
           : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, v, scale, 1)
           : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, v, scale, 2)
                      : __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, v, scale, 3);
  } else {
    const half2_t v = __builtin_bit_cast(half2_t, pair);
    return sel == 0   ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, v, scale, 0)
           : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, v, scale, 1)
           : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, v, scale, 2)
                      : __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, v, scale, 3);
  }
}

// byte pair `SEL` of `w` (two e2m1 codes, low nibble first) * scale -> two 16-bit floats (first value in the low half)
template <int DST>
__device__ __forceinline__ uint32_t cvt_pk_from_fp4(uint32_t w, float scale, int sel) {
  if constexpr (DST == TK_BF16) {
    const bf16x2_t r = sel == 0   ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0)
                       : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1)
                       : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2)
                                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3);
    return __builtin_bit_cast(uint32_t, r);
  } else {
    const f16x2_t r = sel == 0   ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 0)
                      : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 1)
                      : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 2)
                                 : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 3);
    return __builtin_bit_cast(uint32_t, r);
  }
}

template <int KIND>
struct TileGeom {
  static constexpr int BB = KIND == TK_E2M1 ? 16 : 32;  // value bytes per block and column
  static constexpr int NB = 128 / BB;                    // blocks per tile
};

// moves the tile's value bytes and scales between LDS and global memory (TO_GLOBAL) or back
template <int KIND, bool TO_GLOBAL>
__device__ __forceinline__ void tile_move(uint8_t* vals_s, uint8_t* sc_s, uint8_t* gvals, uint8_t* gscales, int64_t o, int64_t col0,
                                          int64_t blk0, int64_t L, int64_t inner, int64_t inner_last) {
  constexpr int BB = TileGeom<KIND>::BB, NB = TileGeom<KIND>::NB;
  const int64_t nblk = L / 32;
  const int64_t line_bytes = KIND == TK_E2M1 ? L / 2 : L;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int q = it * kThreads + threadIdx.x;
    const int col = q >> 3, piece = q & 7;
    const int64_t blk = blk0 + piece * 16 / BB;
    if (col0 + col < inner && blk < nblk) {
      const int64_t line = line_of(o, col0 + col, inner, inner_last);
      uint4* g = reinterpret_cast<uint4*>(gvals + line * line_bytes + blk0 * BB + piece * 16);
      uint4* l = reinterpret_cast<uint4*>(vals_s + tile_row(col) * kTilePitch + piece * 16);
      if (TO_GLOBAL)
        *g = *l;
      else
        *l = *g;
    }
  }
  // scales: a column's NB bytes are contiguous in both places, so one thread moves them in one piece (4 or 8 bytes at
  // any alignment) unless the tile hangs over the end of the axis; single-byte accesses cost an instruction and a
  // memory transaction each
  static_assert(kTileCols == kThreads, "one column per thread");
  {
    const int col = threadIdx.x;
    if (col0 + col < inner && blk0 < nblk) {
      const int64_t line = line_of(o, col0 + col, inner, inner_last);
      uint8_t* g = gscales + line * nblk + blk0;
      uint8_t* l = sc_s + col * NB;
      if (blk0 + NB <= nblk) {
        if (TO_GLOBAL)
          __builtin_memcpy(g, l, NB);
        else
          __builtin_memcpy(l, g, NB);
      } else {
        for (int b = 0; blk0 + b < nblk; ++b) {
          if (TO_GLOBAL)
            g[b] = l[b];
          else
            l[b] = g[b];
        }
      }
    }
  }
}

// Quantises the lane's 32 rows x 4 columns of block `b` (raw[i] = row i, two 16-bit elements per dword) into the
// tile's LDS staging arrays.
template <int SRC, int KIND>
__device__ __forceinline__ void quantise_block_to_lds(const uint2 (&raw)[32], uint8_t* vals_s, uint8_t* sc_s, int c4, int b, int rounding) {
  constexpr int BB = TileGeom<KIND>::BB, NB = TileGeom<KIND>::NB;
    auto elem = [&](int i, int c) __attribute__((always_inline)) {
      const uint32_t w = c < 2 ? raw[i].x : raw[i].y;
      const uint16_t e = (uint16_t)((c & 1) ? (w >> 16) : (w & 0xFFFFu));
      return Elem<SRC>::load(&e);
    };
    // e2m1: the block maxima come from the 16-bit patterns themselves (|x| orders like its bits without the sign, two
    // elements per instruction) and the hardware converts two 16-bit floats to two e2m1 codes while dividing by the
    // power-of-two scale (round to nearest even, saturating at +-6, exact), so a pair of rows costs one byte permute
    // and one conversion.  Blocks that hold an infinity or a NaN, or whose scale is so extreme that subnormal inputs
    // could matter, take the fp32 path below.
    uint32_t max01 = 0, max23 = 0;
    if constexpr (KIND == TK_E2M1) {
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        max01 = pk_max_u16(max01, raw[i].x & 0x7FFF7FFFu);
        max23 = pk_max_u16(max23, raw[i].y & 0x7FFF7FFFu);
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint4* dst = reinterpret_cast<uint4*>(vals_s + tile_row(c4 + c) * kTilePitch + b * BB);
      if constexpr (KIND == TK_E2M1) {
        const uint32_t mx = c < 2 ? max01 : max23;
        const uint32_t m16 = (c & 1) ? (mx >> 16) : (mx & 0xFFFFu);
        const float mf = SRC == TK_BF16 ? hd_bits_f32(m16 << 16) : f16_bits_to_f32((uint16_t)m16);
        const uint32_t sb = mx_scale_bits(mf, KIND, rounding);
        const bool finite = SRC == TK_BF16 ? m16 < 0x7F80u : m16 < 0x7C00u;
        if (finite && sb >= (16u << 23) && sb <= (250u << 23)) {
          const float scale = hd_bits_f32(sb);
          uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < 32; i += 2) {
            const uint32_t lo = c < 2 ? raw[i].x : raw[i].y, hi = c < 2 ? raw[i + 1].x : raw[i + 1].y;
            const uint32_t pair = __builtin_amdgcn_perm(hi, lo, (c & 1) ? 0x07060302u : 0x05040100u);  // (row i, row i+1) of column c
            w[i >> 3] = cvt_pk_fp4<SRC>(w[i >> 3], pair, scale, (i >> 1) & 3);
          }
          dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
          sc_s[(c4 + c) * NB + b] = (uint8_t)(sb >> 23);
          continue;
        }
      }
      float m = 0.0f;
#pragma unroll
      for (int i = 0; i < 32; ++i) m = fmaxf(m, fabsf(elem(i, c)));
      const uint32_t sbits = mx_scale_bits(m, KIND, rounding);
      const float inv = mx_inv_scale(sbits);
      if (KIND == TK_E2M1) {
        // hardware conversion (round to nearest even, saturating at +-6); NaN is first turned into the infinity of
        // its sign so that it saturates like the reference's bit algorithm (mxfp.py:298-327)
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 32; i += 2) {
          float q0 = elem(i, c) * inv, q1 = elem(i + 1, c) * inv;
          q0 = q0 != q0 ? __builtin_copysignf(INFINITY, q0) : q0;
          q1 = q1 != q1 ? __builtin_copysignf(INFINITY, q1) : q1;
          if ((i & 6) == 0) w[i >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[i >> 3], q0, q1, 1.0f, 0);
          if ((i & 6) == 2) w[i >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[i >> 3], q0, q1, 1.0f, 1);
          if ((i & 6) == 4) w[i >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[i >> 3], q0, q1, 1.0f, 2);
          if ((i & 6) == 6) w[i >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[i >> 3], q0, q1, 1.0f, 3);
        }
        dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
      } else {
        uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 32; ++i) w[i >> 2] |= quant_byte<KIND>(elem(i, c) * inv) << (8 * (i & 3));
        dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
        dst[BB / 32] = make_uint4(w[4], w[5], w[6], w[7]);
      }
      sc_s[(c4 + c) * NB + b] = (uint8_t)(sbits >> 23);
    }
}

// 8 bytes of a stream that is read exactly once: the non-temporal hint keeps the lines from displacing what the L2
// still has to merge (the output lines at the tiles' seams); measured 0.281 -> 0.264 ms on [32, 2880, 5760] bf16.
// (The same hint on the dequantiser's row stores costs 5 %: 0.275 -> 0.288 ms.)
__device__ __forceinline__ uint2 load_once_u2(const uint16_t* p) {
  const u32x2_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
  return make_uint2(t.x, t.y);
}

template <int SRC, int KIND>
__global__ __launch_bounds__(kThreads) void mx_down_tile(const uint16_t* __restrict__ src, int64_t stride_outer, int64_t stride_axis,
                                                         int64_t L, int64_t inner, int64_t inner_last, int64_t col_tiles,
                                                         int64_t blk_tiles, uint8_t* __restrict__ out_vals,
                                                         uint8_t* __restrict__ out_scales, int rounding) {
  constexpr int NB = TileGeom<KIND>::NB;
  __shared__ __attribute__((aligned(16))) uint8_t vals_s[kTileRows * kTilePitch];
  __shared__ uint8_t sc_s[kTileCols * NB];
  int64_t bid = tile_order(blockIdx.x, gridDim.x);
  const int64_t bt = bid % blk_tiles;
  bid /= blk_tiles;
  const int64_t ct = bid % col_tiles;
  const int64_t o = bid / col_tiles;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: row addresses stay scalar
  const int64_t col0 = ct * kTileCols, blk0 = bt * NB;
  const int c4 = lane * 4;  // this lane's four columns inside the tile
  if constexpr (NB / 4 == 2) {
    // e2m1 (two blocks per wave): the rows of BOTH blocks are requested before either is converted.  That takes 171
    // registers, so two workgroups share a CU instead of four, each wave with 32 KB on its way instead of 16: measured
    // 0.314 -> 0.281 ms on [32, 2880, 5760] bf16.  (Fewer resident workgroups help on their own, 0.289 ms with the one-block
    // loop held to two waves per SIMD; one wave per SIMD is too few, 0.317 ms.)
    uint2 raw0[32], raw1[32];
    const bool ok0 = blk0 + wave < L / 32 && col0 + c4 < inner, ok1 = blk0 + wave + 4 < L / 32 && col0 + c4 < inner;
    const int64_t bb0 = ok0 ? blk0 + wave : 0, bb1 = ok1 ? blk0 + wave + 4 : bb0;
    const int64_t cc = col0 + c4 < inner ? col0 + c4 : 0;
    const uint16_t* p0 = src + o * stride_outer + bb0 * 32 * stride_axis + cc;
    const uint16_t* p1 = src + o * stride_outer + bb1 * 32 * stride_axis + cc;
#pragma unroll
    for (int i = 0; i < 32; ++i) raw0[i] = load_once_u2(p0 + i * stride_axis);
#pragma unroll
    for (int i = 0; i < 32; ++i) raw1[i] = load_once_u2(p1 + i * stride_axis);
    if (ok0) quantise_block_to_lds<SRC, KIND>(raw0, vals_s, sc_s, c4, wave, rounding);
    if (ok1) quantise_block_to_lds<SRC, KIND>(raw1, vals_s, sc_s, c4, wave + 4, rounding);
  } else
#pragma unroll 1
  for (int pass = 0; pass < NB / 4; ++pass) {
    const int b = wave + 4 * pass;
    if (blk0 + b >= L / 32 || col0 + c4 >= inner) continue;
    const uint16_t* p = src + o * stride_outer + (blk0 + b) * 32 * stride_axis + col0 + c4;
    // the 32 rows stay packed (two 16-bit elements per register) and are widened where they are used: half the
    // registers of an fp32 copy, which is what lets four workgroups share a CU and overlap their load phases
    uint2 raw[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) raw[i] = *reinterpret_cast<const uint2*>(p + i * stride_axis);
    quantise_block_to_lds<SRC, KIND>(raw, vals_s, sc_s, c4, b, rounding);
  }
  __syncthreads();
  tile_move<KIND, true>(vals_s, sc_s, out_vals, out_scales, o, col0, blk0, L, inner, inner_last);
}

template <int KIND, int DST>
__global__ __launch_bounds__(kThreads) void mx_up_tile(const uint8_t* __restrict__ vals, const uint8_t* __restrict__ scales, int64_t L,
                                                       int64_t inner, int64_t inner_last, int64_t col_tiles, int64_t blk_tiles,
                                                       uint16_t* __restrict__ out, int64_t ostride_outer, int64_t ostride_axis) {
  constexpr int BB = TileGeom<KIND>::BB, NB = TileGeom<KIND>::NB;
  __shared__ __attribute__((aligned(16))) uint8_t vals_s[kTileRows * kTilePitch];
  __shared__ uint8_t sc_s[kTileCols * NB];
  int64_t bid = tile_order(blockIdx.x, gridDim.x);
  const int64_t bt = bid % blk_tiles;
  bid /= blk_tiles;
  const int64_t ct = bid % col_tiles;
  const int64_t o = bid / col_tiles;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: row addresses stay scalar
  const int64_t col0 = ct * kTileCols, blk0 = bt * NB;
  const int c4 = lane * 4;
  tile_move<KIND, false>(vals_s, sc_s, const_cast<uint8_t*>(vals), const_cast<uint8_t*>(scales), o, col0, blk0, L, inner, inner_last);
  __syncthreads();
  const float mf = Elem<DST>::max_finite();
#pragma unroll 1
  for (int pass = 0; pass < NB / 4; ++pass) {
    const int b = wave + 4 * pass;
    if (blk0 + b >= L / 32 || col0 + c4 >= inner) continue;
    uint16_t* q = out + o * ostride_outer + (blk0 + b) * 32 * ostride_axis + col0 + c4;
    if constexpr (KIND == TK_E2M1) {
      // Common case, all four blocks of the lane have a scale for which element * scale is a normal number of the
      // target type whatever the element: the hardware conversion (two codes -> two scaled 16-bit floats, exact, no
      // clamp needed) yields rows (i, i+1) of one column, a byte permute per output dword regroups two columns'
      // results into (column c, column c+1) of one row, and every 8 rows are stored as soon as they are complete.
      uint32_t sb4[4];
      bool all_fast = true;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        sb4[c] = sc_s[(c4 + c) * NB + b];
        all_fast = all_fast && (DST == TK_BF16 ? (sb4[c] >= 8 && sb4[c] <= 248) : (sb4[c] >= 114 && sb4[c] <= 139));
      }
      if (all_fast) {
        uint4 w4[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) w4[c] = *reinterpret_cast<const uint4*>(vals_s + tile_row(c4 + c) * kTilePitch + b * BB);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t pr[4][4];  // [column][row pair of this group of 8 rows]
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const uint32_t w = d == 0 ? w4[c].x : d == 1 ? w4[c].y : d == 2 ? w4[c].z : w4[c].w;
            const float scale = hd_bits_f32(sb4[c] << 23);
#pragma unroll
            for (int g = 0; g < 4; ++g) pr[c][g] = cvt_pk_from_fp4<DST>(w, scale, g);
          }
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int i = d * 8 + g * 2;
            *reinterpret_cast<uint2*>(q + i * ostride_axis) =
                make_uint2(__builtin_amdgcn_perm(pr[1][g], pr[0][g], 0x05040100u), __builtin_amdgcn_perm(pr[3][g], pr[2][g], 0x05040100u));
            *reinterpret_cast<uint2*>(q + (i + 1) * ostride_axis) =
                make_uint2(__builtin_amdgcn_perm(pr[1][g], pr[0][g], 0x07060302u), __builtin_amdgcn_perm(pr[3][g], pr[2][g], 0x07060302u));
          }
        }
        continue;
      }
    }
    // general path (fp8 values, or a block with an extreme scale): element by element with the clamp, eight rows at a
    // time so that only those rows' results are held in registers
    uint4 wa[4], wb[4];
    uint32_t sb4g[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint4* srcp = reinterpret_cast<const uint4*>(vals_s + tile_row(c4 + c) * kTilePitch + b * BB);
      wa[c] = srcp[0];
      wb[c] = KIND == TK_E2M1 ? wa[c] : srcp[BB / 32];
      sb4g[c] = sc_s[(c4 + c) * NB + b];
    }
    auto word = [](const uint4& v, int k) __attribute__((always_inline)) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; };
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t hp[8][2];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          float f;
          if (KIND == TK_E2M1) {
            const uint32_t code = (word(wa[c], d) >> (4 * r)) & 0xFu;
            f = mx_dequant(bf16_bits_to_f32((uint16_t)e2m1_to_bf16_bits(code)), sb4g[c], mf, false);
          } else {
            const int k = 2 * d + (r >> 2);  // dword of the block's 32 bytes
            const uint32_t byte = (word(k < 4 ? wa[c] : wb[c], k & 3) >> (8 * (r & 3))) & 0xFFu;
            f = mx_dequant(elem_f32<KIND>(byte), sb4g[c], mf, KIND == TK_E5M2);
          }
          uint16_t e;
          Elem<DST>::store(&e, f);
          if (c & 1)
            hp[r][c >> 1] |= (uint32_t)e << 16;
          else
            hp[r][c >> 1] = e;
        }
      }
#pragma unroll
      for (int r = 0; r < 8; ++r) *reinterpret_cast<uint2*>(q + (d * 8 + r) * ostride_axis) = make_uint2(hp[r][0], hp[r][1]);
    }
  }
}

// ---- dispatch helpers --------------------------------------------------------------------------
template <int SRC, int KIND>
int32_t launch_down(const void* src, int64_t outer, int64_t L, int64_t inner, int64_t inner_last, int64_t so, int64_t sa, int64_t si,
                    void* out_vals, void* out_scales, int rounding, hipStream_t st) {
  typedef typename Elem<SRC>::T T;
  const T* s = static_cast<const T*>(src);
  uint8_t* ov = static_cast<uint8_t*>(out_vals);
  uint8_t* os = static_cast<uint8_t*>(out_scales);
  if (inner == 1 && sa == 1) {
    // rows = outer, row stride = so
    const int64_t total = outer * (L / 8);
    const int64_t grid = cdiv(total, kThreads);
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_downcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_down_rows<SRC, KIND>), dim3((unsigned)grid), dim3(kThreads), 0, st, s, so, outer, L, ov, os,
                       rounding);
    return check_launch("mx_down_rows");
  }
  if (si != 1 && inner != 1) return fail(TK_ERR_UNSUPPORTED, "tk_mx_downcast: inner stride must be 1");
  const int64_t nblk = L / 32;
  if constexpr (sizeof(T) == 2) {
    if (inner % 4 == 0 && sa % 4 == 0 && so % 4 == 0 && (reinterpret_cast<uintptr_t>(src) % 8) == 0 &&
        (reinterpret_cast<uintptr_t>(out_vals) % 16) == 0) {
      const int64_t col_tiles = cdiv(inner, kTileCols), blk_tiles = cdiv(nblk, TileGeom<KIND>::NB);
      const int64_t grid = col_tiles * blk_tiles * outer;
      if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_downcast: tensor too large for one launch");
      hipLaunchKernelGGL((mx_down_tile<SRC, KIND>), dim3((unsigned)grid), dim3(kThreads), 0, st, reinterpret_cast<const uint16_t*>(s), so, sa,
                         L, inner, inner_last, col_tiles, blk_tiles, ov, os, rounding);
      return check_launch("mx_down_tile");
    }
  }
  const int64_t blk_tiles = cdiv(nblk, 4);
  const size_t esz = sizeof(T);
  const bool pair_ok = inner % 2 == 0 && sa % 2 == 0 && so % 2 == 0 && (reinterpret_cast<uintptr_t>(src) % (2 * esz)) == 0;
  if (pair_ok) {
    const int64_t col_tiles = cdiv(inner, 128);
    const int64_t grid = col_tiles * blk_tiles * outer;
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_downcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_down_cols<SRC, KIND, 2>), dim3((unsigned)grid), dim3(kThreads), 0, st, s, so, sa, L, inner,
                       inner_last, col_tiles, blk_tiles, ov, os, rounding);
  } else {
    const int64_t col_tiles = cdiv(inner, 64);
    const int64_t grid = col_tiles * blk_tiles * outer;
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_downcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_down_cols<SRC, KIND, 1>), dim3((unsigned)grid), dim3(kThreads), 0, st, s, so, sa, L, inner,
                       inner_last, col_tiles, blk_tiles, ov, os, rounding);
  }
  return check_launch("mx_down_cols");
}

template <int KIND, int DST>
int32_t launch_up(const void* vals, const void* scales, int64_t outer, int64_t L, int64_t inner, int64_t inner_last, void* out, int64_t oso,
                  int64_t osa, int64_t osi, hipStream_t st) {
  typedef typename Elem<DST>::T T;
  const uint8_t* v = static_cast<const uint8_t*>(vals);
  const uint8_t* s = static_cast<const uint8_t*>(scales);
  T* o = static_cast<T*>(out);
  if (inner == 1 && osa == 1) {
    const int64_t total = outer * (L / 8);
    const int64_t grid = cdiv(total, kThreads);
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_upcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_up_rows<KIND, DST>), dim3((unsigned)grid), dim3(kThreads), 0, st, v, s, outer, L, o, oso);
    return check_launch("mx_up_rows");
  }
  if (osi != 1 && inner != 1) return fail(TK_ERR_UNSUPPORTED, "tk_mx_upcast: output inner stride must be 1");
  const int64_t nblk = L / 32;
  if constexpr (sizeof(T) == 2) {
    if (inner % 4 == 0 && osa % 4 == 0 && oso % 4 == 0 && (reinterpret_cast<uintptr_t>(out) % 8) == 0 &&
        (reinterpret_cast<uintptr_t>(vals) % 16) == 0) {
      const int64_t col_tiles = cdiv(inner, kTileCols), blk_tiles = cdiv(nblk, TileGeom<KIND>::NB);
      const int64_t grid = col_tiles * blk_tiles * outer;
      if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_upcast: tensor too large for one launch");
      hipLaunchKernelGGL((mx_up_tile<KIND, DST>), dim3((unsigned)grid), dim3(kThreads), 0, st, v, s, L, inner, inner_last, col_tiles,
                         blk_tiles, reinterpret_cast<uint16_t*>(o), oso, osa);
      return check_launch("mx_up_tile");
    }
  }
  const int64_t blk_tiles = cdiv(nblk, 4);
  const size_t esz = sizeof(T);
  const bool pair_ok = inner % 2 == 0 && osa % 2 == 0 && oso % 2 == 0 && (reinterpret_cast<uintptr_t>(out) % (2 * esz)) == 0;
  if (pair_ok) {
    const int64_t col_tiles = cdiv(inner, 128);
    const int64_t grid = col_tiles * blk_tiles * outer;
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_upcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_up_cols<KIND, DST, 2>), dim3((unsigned)grid), dim3(kThreads), 0, st, v, s, L, inner,
                       inner_last, col_tiles, blk_tiles, o, oso, osa);
  } else {
    const int64_t col_tiles = cdiv(inner, 64);
    const int64_t grid = col_tiles * blk_tiles * outer;
    if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_mx_upcast: tensor too large for one launch");
    hipLaunchKernelGGL((mx_up_cols<KIND, DST, 1>), dim3((unsigned)grid), dim3(kThreads), 0, st, v, s, L, inner,
                       inner_last, col_tiles, blk_tiles, o, oso, osa);
  }
  return check_launch("mx_up_cols");
}

}  // namespace
}  // namespace tk

using namespace tk;

extern "C" int32_t tk_mx_downcast(const void* src, int32_t src_dtype, int64_t outer, int64_t axis_len, int64_t inner,
                                  int64_t inner_last, int64_t stride_outer, int64_t stride_axis, int64_t stride_inner, void* out_vals,
                                  void* out_scales, int32_t out_kind, int32_t rounding, tk_stream_t stream) {
  if (outer < 0 || axis_len < 0 || inner < 0) return fail(TK_ERR_INVALID, "tk_mx_downcast: negative size");
  if (axis_len % 32 != 0) return fail(TK_ERR_INVALID, "tk_mx_downcast: axis length %lld is not a multiple of 32", (long long)axis_len);
  if (rounding != TK_MX_ROUND_UP && rounding != TK_MX_ROUND_DOWN) return fail(TK_ERR_INVALID, "tk_mx_downcast: bad rounding mode %d", rounding);
  if (out_kind != TK_E2M1 && out_kind != TK_E4M3 && out_kind != TK_E5M2) return fail(TK_ERR_INVALID, "tk_mx_downcast: bad output kind %d", out_kind);
  if (outer == 0 || axis_len == 0 || inner == 0) return TK_OK;
  if (inner_last <= 0 || inner % inner_last != 0) return fail(TK_ERR_INVALID, "tk_mx_downcast: inner_last must divide inner");
  if (!src || !out_vals || !out_scales) return fail(TK_ERR_INVALID, "tk_mx_downcast: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
#define TK_DOWN(S, K) \
  if (src_dtype == S && out_kind == K) return launch_down<S, K>(src, outer, axis_len, inner, inner_last, stride_outer, stride_axis, stride_inner, out_vals, out_scales, rounding, st);
  TK_DOWN(TK_BF16, TK_E2M1)
  TK_DOWN(TK_BF16, TK_E4M3)
  TK_DOWN(TK_BF16, TK_E5M2)
  TK_DOWN(TK_F16, TK_E2M1)
  TK_DOWN(TK_F16, TK_E4M3)
  TK_DOWN(TK_F16, TK_E5M2)
  TK_DOWN(TK_F32, TK_E2M1)
  TK_DOWN(TK_F32, TK_E4M3)
  TK_DOWN(TK_F32, TK_E5M2)
#undef TK_DOWN
  return fail(TK_ERR_INVALID, "tk_mx_downcast: unsupported source dtype %d", src_dtype);
}

extern "C" int32_t tk_mx_upcast(const void* vals, const void* scales, int32_t kind, int64_t outer, int64_t axis_len,
                                int64_t inner, int64_t inner_last, void* out, int32_t out_dtype, int64_t ostride_outer,
                                int64_t ostride_axis, int64_t ostride_inner, tk_stream_t stream) {
  if (outer < 0 || axis_len < 0 || inner < 0) return fail(TK_ERR_INVALID, "tk_mx_upcast: negative size");
  if (axis_len % 32 != 0) return fail(TK_ERR_INVALID, "tk_mx_upcast: axis length %lld is not a multiple of 32", (long long)axis_len);
  if (kind != TK_E2M1 && kind != TK_E4M3 && kind != TK_E5M2) return fail(TK_ERR_INVALID, "tk_mx_upcast: bad element kind %d", kind);
  if (outer == 0 || axis_len == 0 || inner == 0) return TK_OK;
  if (inner_last <= 0 || inner % inner_last != 0) return fail(TK_ERR_INVALID, "tk_mx_upcast: inner_last must divide inner");
  if (!vals || !scales || !out) return fail(TK_ERR_INVALID, "tk_mx_upcast: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
#define TK_UP(K, D) \
  if (kind == K && out_dtype == D) return launch_up<K, D>(vals, scales, outer, axis_len, inner, inner_last, out, ostride_outer, ostride_axis, ostride_inner, st);
  TK_UP(TK_E2M1, TK_BF16)
  TK_UP(TK_E2M1, TK_F16)
  TK_UP(TK_E2M1, TK_F32)
  TK_UP(TK_E4M3, TK_BF16)
  TK_UP(TK_E4M3, TK_F16)
  TK_UP(TK_E4M3, TK_F32)
  TK_UP(TK_E5M2, TK_BF16)
  TK_UP(TK_E5M2, TK_F16)
  TK_UP(TK_E5M2, TK_F32)
#undef TK_UP
  return fail(TK_ERR_INVALID, "tk_mx_upcast: unsupported output dtype %d", out_dtype);
}
