// GEMM whose REDUCTION dimension is ragged (the expert weight gradient of a MoE layer):
//   y[e, m, n] = sum over k < sizes[e] of a[m, a_offs[e] + k] * b[b_offs[e] + k, n]
// Follows tk/matmul.py:376-384 (`b_ragged_metadata` selects ragged_dimension "K", one output per slice),
// tk/matmul_details/_matmul.py:252-272 (a slice's k range comes from the slice offsets of BOTH operands, its length
// from the slice sizes) and the torch statement of it in tk/matmul.py:852-875.
//
// In the weight-gradient use a = x^T [hidden, rows] and b = dy [rows, n] are both stored with the reduction index as
// the SLOW dimension, while an MFMA lane wants 8 consecutive k of one row.  The transposition happens between the
// global load and LDS: a thread fetches four k rows of the same eight m (four 16-byte loads, coalesced along m),
// interleaves them in registers and writes eight 8-byte pieces [m][k..k+3]; the MFMA operands are then plain
// 16-byte LDS reads.  An operand stored k-contiguous skips the interleave.  Anything that is not 16-byte aligned or
// hangs over an edge takes an element-wise path with zero fill (k past the slice MUST read as zero: the neighbouring
// rows belong to another expert).
//
// The problem is bound by writing y (n_slices * M * N outputs from short reductions), not by the MFMAs: at 128
// experts x 2880 x 5760 from 256 rows each the output is 4.2 GB against 1.1 TFLOP.
#include <type_traits>

#include "common.h"

namespace tk {
namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

struct RaggedKParams {
  const uint8_t* a;
  int64_t a_stride_m, a_stride_k;  // elements
  const uint8_t* b;
  int64_t b_stride_k, b_stride_n;
  uint8_t* y;
  int64_t y_stride_e, y_stride_m;
  const int32_t* sizes;
  const int32_t* a_offs;
  const int32_t* b_offs;
  int M, N;
  int tiles_m, tiles_n;
  int y_dtype;
  uint32_t a_bytes, b_bytes;  // extents for the buffer resources of the fast variant
  int a_vec, b_vec;  // the operand's base and strides allow 16-byte loads along its contiguous dimension
};

constexpr int kTile = 128;  // output tile edge (rows and columns)
constexpr int kKC = 32;     // k per pipeline stage
constexpr int kRing = 3;   // stages of global loads in flight per thread
constexpr int kPitch = kKC * 2 + 16;  // bytes per LDS row: 32 k + a pad that keeps 16-byte alignment and spreads banks

template <class F>
__device__ __forceinline__ void static_for_ring(F&& f) {
  f(std::integral_constant<int, 0>{});
  f(std::integral_constant<int, 1>{});
  f(std::integral_constant<int, 2>{});
  static_assert(kRing == 3, "static_for_ring lists the slots");
}

// FAST: both operands are stored with the reduction index slow, 16-byte loads are possible everywhere and M and N are
// multiples of 8 (so a thread's eight rows are all inside or all outside).  The loads then go through a buffer
// resource with an out-of-range offset for pieces past the slice end or the matrix edge (the hardware returns zeros),
// so no branch surrounds a load and the compiler's wait counts let all kRing stages stay in flight.
template <int DT, bool FAST>
__global__ __launch_bounds__(256) void ragged_k_gemm_kernel(const RaggedKParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][kTile * kPitch];  // [buffer][operand][row][k]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, h = lane >> 5;
  const int mw = wave & 1, nw = wave >> 1;  // the wave's 64 x 64 quadrant

  // workgroups go round-robin to the 8 XCDs; renumber so that consecutive tiles, which share a slice's operand rows,
  // run on one XCD and find them in its L2
  int pid;
  {
    const int total = gridDim.x, per = total / 8, extra = total % 8;
    const int grp = blockIdx.x % 8, local = blockIdx.x / 8;
    pid = grp * per + (grp < extra ? grp : extra) + local;
  }
  const int tn = pid % p.tiles_n;
  pid /= p.tiles_n;
  const int tm = pid % p.tiles_m;
  const int e = pid / p.tiles_m;
  const int ksz = p.sizes[e];
  const int a_k0 = p.a_offs[e], b_k0 = p.b_offs[e];
  const int m0 = tm * kTile, n0 = tn * kTile;

  // ---- this thread's piece of a stage: threads 0..127 stage operand a, 128..255 operand b ----
  const bool is_b = tid >= 128;
  const int t7 = tid & 127;
  const uint8_t* base = is_b ? p.b : p.a;
  const int64_t stride_r = is_b ? p.b_stride_n : p.a_stride_m;
  const int64_t stride_k = is_b ? p.b_stride_k : p.a_stride_k;
  const int k_first = is_b ? b_k0 : a_k0;
  const int r0 = is_b ? n0 : m0;
  const int rows_total = is_b ? p.N : p.M;
  const bool vec_ok = (is_b ? p.b_vec : p.a_vec) != 0;
  const bool k_slow = stride_r == 1;
  // k-slow: piece = 4 k rows (kq*4 ..) x 8 rows (rb*8 ..);  k-contiguous: piece = one row x 32 k
  // kq runs fastest over the lanes: the eight lanes of one row block write 64 contiguous bytes of an LDS row, and row
  // blocks (8 rows = 640 bytes apart) alternate between two bank phases, so an LDS write sees a 2-way conflict at most
  // (with the row block fastest, sixteen lanes would share each bank); a load instruction still covers whole 128-byte
  // lines (8 lanes x 16 bytes along m)
  const int rb = t7 >> 3, kq = t7 & 7;
  // staged registers, a ring of kRing stages: k-slow 4 x uint4 = [k][8 rows]; k-contiguous 4 x uint4 = 32 k of one row
  uint32_t ring[kRing][16];
  uint8_t* my_lds0 = &lds[0][is_b ? 1 : 0][0];

  auto load_elem = [&](int64_t r, int64_t k) __attribute__((always_inline)) -> uint32_t {
    return *reinterpret_cast<const uint16_t*>(base + ((r0 + r) * stride_r + (k_first + k) * stride_k) * 2);
  };
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(is_b ? p.b : p.a), 0,
                                                                        is_b ? p.b_bytes : p.a_bytes, 0x00020000);
  // byte offset of this thread's eight rows at k = 0 of the slice; kOutOfRange when the rows lie past the edge
  constexpr uint32_t kOutOfRange = 0x80000000u;
  const bool rows_in = r0 + rb * 8 < rows_total;
  const uint32_t off0 = (uint32_t)(((int64_t)(r0 + rb * 8) + (int64_t)k_first * stride_k) * 2);
  const uint32_t kstep = (uint32_t)(stride_k * 2);
  auto load_stage = [&](auto slot_c, int kc) __attribute__((always_inline)) {
    uint32_t(&pr)[16] = ring[decltype(slot_c)::value];
    if constexpr (FAST) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = kc + kq * 4 + q;
        const uint32_t off = (rows_in && k < ksz) ? off0 + (uint32_t)k * kstep : kOutOfRange;
        const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
        pr[4 * q + 0] = v.x;
        pr[4 * q + 1] = v.y;
        pr[4 * q + 2] = v.z;
        pr[4 * q + 3] = v.w;
      }
      return;
    }
    if (k_slow) {
      const int rr = rb * 8;
      const bool full_rows = r0 + rr + 8 <= rows_total;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = kc + kq * 4 + q;
        if (k < ksz && vec_ok && full_rows) {
          const uint4 v = *reinterpret_cast<const uint4*>(base + ((int64_t)(r0 + rr) + (int64_t)(k_first + k) * stride_k) * 2);
          pr[4 * q + 0] = v.x;
          pr[4 * q + 1] = v.y;
          pr[4 * q + 2] = v.z;
          pr[4 * q + 3] = v.w;
        } else {
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            uint32_t lo = 0, hi = 0;
            if (k < ksz) {
              if (r0 + rr + 2 * d < rows_total) lo = load_elem(rr + 2 * d, k);
              if (r0 + rr + 2 * d + 1 < rows_total) hi = load_elem(rr + 2 * d + 1, k);
            }
            pr[4 * q + d] = lo | (hi << 16);
          }
        }
      }
    } else {
      const int r = t7;
      const bool row_ok = r0 + r < rows_total;
      const uint8_t* rowp = base + ((int64_t)(r0 + r) * stride_r + (int64_t)k_first * stride_k) * 2;
      // 16-byte loads need k contiguous, the row start 16-byte aligned (the slice offset decides) and a full piece
      const bool can_vec = vec_ok && stride_k == 1 && row_ok && ((reinterpret_cast<uintptr_t>(rowp) & 15) == 0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = kc + q * 8;
        if (can_vec && k + 8 <= ksz) {
          const uint4 v = *reinterpret_cast<const uint4*>(rowp + (int64_t)k * 2);
          pr[4 * q + 0] = v.x;
          pr[4 * q + 1] = v.y;
          pr[4 * q + 2] = v.z;
          pr[4 * q + 3] = v.w;
        } else {
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            uint32_t lo = 0, hi = 0;
            if (row_ok) {
              if (k + 2 * d < ksz) lo = load_elem(r, k + 2 * d);
              if (k + 2 * d + 1 < ksz) hi = load_elem(r, k + 2 * d + 1);
            }
            pr[4 * q + d] = lo | (hi << 16);
          }
        }
      }
    }
  };
  auto store_stage = [&](auto slot_c, int buf) __attribute__((always_inline)) {
    uint32_t(&pr)[16] = ring[decltype(slot_c)::value];
    uint8_t* dst = my_lds0 + buf * (2 * kTile * kPitch);
    if (FAST || k_slow) {
      // pr[4q + d] = rows (2d, 2d+1) at k = kq*4 + q  ->  row i gets its four k as one 8-byte piece
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t a0 = pr[d], a1 = pr[4 + d], a2 = pr[8 + d], a3 = pr[12 + d];
        const uint2 even = make_uint2((a0 & 0xFFFFu) | (a1 << 16), (a2 & 0xFFFFu) | (a3 << 16));
        const uint2 odd = make_uint2((a0 >> 16) | (a1 & 0xFFFF0000u), (a2 >> 16) | (a3 & 0xFFFF0000u));
        *reinterpret_cast<uint2*>(dst + (rb * 8 + 2 * d) * kPitch + kq * 8) = even;
        *reinterpret_cast<uint2*>(dst + (rb * 8 + 2 * d + 1) * kPitch + kq * 8) = odd;
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<uint4*>(dst + t7 * kPitch + q * 16) = make_uint4(pr[4 * q], pr[4 * q + 1], pr[4 * q + 2], pr[4 * q + 3]);
    }
  };

  f32x16_t acc[2][2];  // [n fragment][m fragment]
#pragma unroll
  for (int f = 0; f < 2; ++f)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[f][j][i] = 0.f;

  auto compute = [&](int buf) __attribute__((always_inline)) {
    const uint8_t* am = &lds[buf][0][0] + (mw * 64 + lr) * kPitch;
    const uint8_t* bn = &lds[buf][1][0] + (nw * 64 + lr) * kPitch;
#pragma unroll
    for (int t = 0; t < kKC / 16; ++t) {
      uint4 af[2], bf[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) af[j] = *reinterpret_cast<const uint4*>(am + j * 32 * kPitch + (t * 16 + h * 8) * 2);
#pragma unroll
      for (int f = 0; f < 2; ++f) bf[f] = *reinterpret_cast<const uint4*>(bn + f * 32 * kPitch + (t * 16 + h * 8) * 2);
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          // first operand = the output COLUMN side: accumulator register i of lane (lr, h) is then column
          // (i >> 2) * 8 + h * 4 + (i & 3) of row lr, four consecutive columns per register quad
          if constexpr (DT == TK_BF16)
            acc[f][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[f]), __builtin_bit_cast(bf16x8_t, af[j]),
                                                                acc[f][j], 0, 0, 0);
          else
            acc[f][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, bf[f]), __builtin_bit_cast(f16x8_t, af[j]),
                                                               acc[f][j], 0, 0, 0);
        }
    }
  };

  // The slices are short (a few hundred k at most), so a tile is a handful of stages and the global-load latency is
  // what it costs: the loads run kRing stages ahead in registers, the LDS copy one stage ahead (two LDS buffers, one
  // barrier per stage).
  const int nstages = (ksz + kKC - 1) / kKC;
  if (nstages > 0) {
    static_for_ring([&](auto i_c) __attribute__((always_inline)) {
      if (decltype(i_c)::value < nstages) load_stage(i_c, decltype(i_c)::value * kKC);
    });
    store_stage(std::integral_constant<int, 0>{}, 0);
    __syncthreads();
    for (int c = 0; c < nstages; c += kRing) {
      static_for_ring([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        const int cc = c + i;
        if (cc < nstages) {  // uniform
          if (cc + 1 < nstages) store_stage(std::integral_constant<int, (i + 1) % kRing>{}, (cc + 1) & 1);
          if (cc + kRing < nstages) load_stage(i_c, (cc + kRing) * kKC);  // slot i went to LDS one stage ago
          compute(cc & 1);
          __syncthreads();
        }
      });
    }
  }

  // ---- store ----
  // A lane's accumulator quad is four columns of ONE row and the 32 lanes of a fragment are 32 different rows, so
  // direct stores would touch 32 cache lines with 16 bytes each per instruction.  Instead a wave passes each 32-row
  // half of its quadrant through its own slice of LDS (the operand buffers are free now) and writes whole rows:
  // 128 bytes (16-bit outputs) or 256 bytes (fp32) of a row per 8 or 16 lanes.
  const int esize = p.y_dtype == TK_F32 ? 4 : 2;
  uint8_t* ye = p.y + (int64_t)e * p.y_stride_e * esize;
  const bool y_vec = ((p.y_stride_m * esize) % 16 == 0) && ((reinterpret_cast<uintptr_t>(ye) & 15) == 0);
  constexpr int kStagePitch = 64 * 4 + 16;  // bytes per staged row (64 columns of up to 4 bytes + pad)
  static_assert(4 * 32 * kStagePitch <= (int)sizeof(lds), "staging fits the operand buffers");
  uint8_t* stage = &lds[0][0][0] + wave * 32 * kStagePitch;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int col = f * 32 + u * 8 + h * 4;  // within the wave's 64 columns
        const float vv[4] = {acc[f][j][4 * u], acc[f][j][4 * u + 1], acc[f][j][4 * u + 2], acc[f][j][4 * u + 3]};
        if (p.y_dtype == TK_F32) {
          *reinterpret_cast<float4*>(stage + lr * kStagePitch + col * 4) = make_float4(vv[0], vv[1], vv[2], vv[3]);
        } else {
          uint32_t b[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) b[i] = p.y_dtype == TK_BF16 ? f32_to_bf16_bits(vv[i]) : f32_to_f16_bits(vv[i]);
          *reinterpret_cast<uint2*>(stage + lr * kStagePitch + col * 2) = make_uint2(b[0] | (b[1] << 16), b[2] | (b[3] << 16));
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int lanes_per_row = 64 * esize / 16;  // 8 or 16
    const int rows_per_it = 64 / lanes_per_row;
    const int piece = lane % lanes_per_row;
    const int ncol = n0 + nw * 64 + piece * (16 / esize);
    for (int it = 0; it < 32 / rows_per_it; ++it) {
      const int r = it * rows_per_it + lane / lanes_per_row;
      const int m = m0 + mw * 64 + j * 32 + r;
      if (m >= p.M || ncol >= p.N) continue;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + r * kStagePitch + piece * 16);
      uint8_t* dst = ye + ((int64_t)m * p.y_stride_m + ncol) * esize;
      if (y_vec && ncol + 16 / esize <= p.N) {
        *reinterpret_cast<uint4*>(dst) = v;
      } else {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        for (int i = 0; i < 16 / esize && ncol + i < p.N; ++i) {
          if (esize == 4)
            reinterpret_cast<uint32_t*>(dst)[i] = w[i];
          else
            reinterpret_cast<uint16_t*>(dst)[i] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

}  // namespace
}  // namespace tk

extern "C" int32_t tk_ragged_k_gemm(const tk_ragged_k_desc* d, tk_stream_t stream) {
  using namespace tk;
  if (!d) return fail(TK_ERR_INVALID, "tk_ragged_k_gemm: null descriptor");
  if (d->dtype != TK_BF16 && d->dtype != TK_F16) return fail(TK_ERR_UNSUPPORTED, "tk_ragged_k_gemm: operands must be bf16 or fp16");
  if (d->y_dtype != TK_BF16 && d->y_dtype != TK_F16 && d->y_dtype != TK_F32)
    return fail(TK_ERR_UNSUPPORTED, "tk_ragged_k_gemm: output must be bf16, fp16 or fp32");
  if (d->M < 0 || d->N < 0 || d->n_slices < 0) return fail(TK_ERR_INVALID, "tk_ragged_k_gemm: negative size");
  if (d->M == 0 || d->N == 0 || d->n_slices == 0) return TK_OK;
  if (!d->a || !d->b || !d->y || !d->slice_sizes || !d->a_slice_offs || !d->b_slice_offs)
    return fail(TK_ERR_INVALID, "tk_ragged_k_gemm: null operand");
  RaggedKParams p;
  p.a = static_cast<const uint8_t*>(d->a);
  p.a_stride_m = d->a_stride_m;
  p.a_stride_k = d->a_stride_k;
  p.b = static_cast<const uint8_t*>(d->b);
  p.b_stride_k = d->b_stride_k;
  p.b_stride_n = d->b_stride_n;
  p.y = static_cast<uint8_t*>(d->y);
  p.y_stride_e = d->y_stride_e;
  p.y_stride_m = d->y_stride_m;
  p.sizes = d->slice_sizes;
  p.a_offs = d->a_slice_offs;
  p.b_offs = d->b_slice_offs;
  p.M = d->M;
  p.N = d->N;
  p.tiles_m = (int)cdiv(d->M, kTile);
  p.tiles_n = (int)cdiv(d->N, kTile);
  p.y_dtype = d->y_dtype;
  // 16-byte loads along the contiguous dimension: base aligned and the other stride a multiple of 8 elements
  auto vec = [](const void* ptr, int64_t s_contig, int64_t s_other) {
    return s_contig == 1 && s_other % 8 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 15) == 0;
  };
  p.a_vec = vec(d->a, d->a_stride_m == 1 ? d->a_stride_m : d->a_stride_k, d->a_stride_m == 1 ? d->a_stride_k : d->a_stride_m);
  p.b_vec = vec(d->b, d->b_stride_n == 1 ? d->b_stride_n : d->b_stride_k, d->b_stride_n == 1 ? d->b_stride_k : d->b_stride_n);
  const int64_t grid = (int64_t)d->n_slices * p.tiles_m * p.tiles_n;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_ragged_k_gemm: grid too large");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // extents (bytes from the base to one past the last element) when both operands are k-slow and within 2 GiB
  const bool k_slow_both = d->a_stride_m == 1 && d->b_stride_n == 1 && d->a_stride_k > 0 && d->b_stride_k > 0;
  const int64_t a_extent = d->a_k_extent * d->a_stride_k * 2, b_extent = d->b_k_extent * d->b_stride_k * 2;
  const bool fast = k_slow_both && p.a_vec && p.b_vec && d->M % 8 == 0 && d->N % 8 == 0 && d->a_k_extent > 0 && d->b_k_extent > 0 &&
                    a_extent < (int64_t(1) << 31) && b_extent < (int64_t(1) << 31) && d->M <= d->a_stride_k && d->N <= d->b_stride_k;
  p.a_bytes = fast ? (uint32_t)a_extent : 0;
  p.b_bytes = fast ? (uint32_t)b_extent : 0;
  auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), 0, st, p); };
  if (d->dtype == TK_BF16) {
    if (fast)
      launch(ragged_k_gemm_kernel<TK_BF16, true>);
    else
      launch(ragged_k_gemm_kernel<TK_BF16, false>);
  } else {
    if (fast)
      launch(ragged_k_gemm_kernel<TK_F16, true>);
    else
      launch(ragged_k_gemm_kernel<TK_F16, false>);
  }
  return check_launch("ragged_k_gemm_kernel");
}
