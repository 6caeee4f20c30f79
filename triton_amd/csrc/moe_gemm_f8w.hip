#include "gemm_common.h"

namespace tk {
namespace {

// ------------------------------------------------------------------------------------------------
// e4m3 weights in the tile-native layout x e4m3 activations, 256 x 256 tiles (large prefill problems)
// ------------------------------------------------------------------------------------------------
// Same operands, layouts and instruction as moe_gemm_f8n_kernel (v_mfma_f32_32x32x64_f8f6f4 on 32 consecutive k bytes
// per lane of both operands; weights global memory -> registers, gathered activation rows through an LDS double buffer),
// with a tile of 256 rows instead of 128.  What bounds the 128-row kernel is the bytes that enter a CU per MFMA: a K-stage
// of 256 bytes brings 32 KB of activations and 64 KB of weights for 2,048 MFMA cycles, and a CU takes in about 26 bytes
// per cycle, so the matrix pipe is busy 0.56 of the time.  256 rows bring 64 + 64 KB for 4,096 MFMA cycles.
//
// A wave owns 64 columns (two fragments) and all eight row fragments: 256 accumulator registers, which are the whole
// accumulation file, so the operands have to live in what is left:
//   * weights: ONE set of registers per stage (64); the registers of K-step t are refilled with the next stage's K-step t
//     as soon as step t has issued its MFMAs, three steps (about 3,000 cycles) before they are used again;
//   * activation fragments: a ring of four (32 registers) instead of a double buffer of eight; the fragment of an MFMA
//     pair is read from LDS two pairs ahead;
//   * staging of the next stage's activations: 16 pieces per thread, written to LDS four per K-step and refilled with the
//     stage after (64 registers, a full stage ahead of their use).
// One workgroup barrier per stage sits in front of the first LDS read that belongs to the next stage's buffer (two pairs
// before the stage ends): by then every wave has issued its last read of the current buffer and written its share of
// the next one (steps 0..3, pairs 0..27).
// All eight row fragments are always multiplied (rows past a block's end repeat its last row and are not stored), so the
// kernel is for row blocks that are mostly full; the host picks it from 512 rows per slice on.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void moe_gemm_f8w_kernel(const GemmParams p) {
  typedef Frag<32> FR;
  constexpr int FM = 32, MFW = 8, NFW = 2, BLKM = 256, BM = 256, BN = 256, KC = 256, NS = 4;
  constexpr int XPITCH = KC + 16;
  constexpr int XBYTES = BM * XPITCH;
  constexpr int XCH = 16;  // 16-byte activation pieces per thread per stage
  constexpr int RING = 4;  // activation fragments in registers
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nw = __builtin_amdgcn_readfirstlane(tid >> 6);  // column quarter of the tile
  const int lr = lane & 31, h = lane >> 5;
  const int K = p.K, N = p.N;
  const int nst = p.w_nst;  // stages of 256
  const int grid = (int)gridDim.x;
  const int live = p.slice_sizes ? p.block_offs[p.n_slices] * p.grid_n : p.total_tiles;
  const int xc = tid & 15;
  const int xlds0 = (tid >> 4) * XPITCH + xc * 16;  // piece j at xlds0 + j*16*XPITCH
  const uint32_t lane16 = lane * 16;
  const int nfr = (N + 31) >> 5;

  // tiles in static rounds, (expert, column tile, row block) order: tiles that start together walk K in step and meet each
  // other's operands in the XCD's L2
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

    // ---- activation staging: piece j of this thread = row 16 j + tid/16, 16-byte chunk tid%16 of the stage; rows are
    // addressed by 32-bit byte offsets from x (the host keeps x below 4 GiB) ----
    uint32_t xoff[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      int row = blk_off + (tid >> 4) + 16 * j;
      row = row < eM ? row : eM - 1;
      const uint32_t src = p.gather ? (uint32_t)p.gather[start_m + row] : (uint32_t)(start_m + row);
      xoff[j] = src * (uint32_t)p.x_stride_m;
    }
    const uint8_t* wbase[NFW];  // uniform
#pragma unroll
    for (int f = 0; f < NFW; ++f) {
      int F = pid_n * (BN / 32) + nw * NFW + f;
      F = F < nfr ? F : nfr - 1;  // fragments past N repeat the last one; their columns are dropped in the epilogue
      wbase[f] = p.w + (int64_t)expert * p.w_stride_e + (int64_t)F * nst * 8192;
    }

    // (two arrays of four row fragments each, rows 0..127 and 128..255 of the tile: the shared epilogue is instantiated for
    // four, as in the 128-row kernel, and one array of eight was left in scratch memory by the compiler)
    typename FR::acc_t acc_lo[NFW][MFW / 2], acc_hi[NFW][MFW / 2];
#pragma unroll
    for (int f = 0; f < NFW; ++f)
#pragma unroll
      for (int j = 0; j < MFW / 2; ++j)
#pragma unroll
        for (int i = 0; i < FR::NACC; ++i) acc_lo[f][j][i] = acc_hi[f][j][i] = 0.f;

    u32x4_t xreg[XCH];
    i32x8_t wreg[NFW][NS];  // [column fragment][K-step]
    i32x8_t xf[RING];       // fragment of pair g (K-step g / 8, row fragment g % 8) in slot g % RING

    // Loads are unconditional: rows past the last valid row re-read it, k past K re-reads the row's last 16 bytes (the
    // padded weights there are zero), stages past the last one re-read the last stage.
    auto load_x_piece = [&](int j, int s) __attribute__((always_inline)) {
      int k0 = s * KC + xc * 16;
      k0 = k0 < K - 16 ? k0 : K - 16;
      xreg[j] = *reinterpret_cast<const u32x4_t*>(p.x + (xoff[j] + (uint32_t)k0));
    };
    auto store_x_piece = [&](int j, int buf) __attribute__((always_inline)) {
      *reinterpret_cast<u32x4_t*>(lds + buf * XBYTES + xlds0 + j * 16 * XPITCH) = xreg[j];
    };
    auto load_w = [&](int f, int t, int s) __attribute__((always_inline)) {
      s = s < nst ? s : nst - 1;
      const uint8_t* a = wbase[f] + (int64_t)s * 8192 + t * 2048 + lane16;
      const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
      const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 1024);
      wreg[f][t] = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    auto read_xf = [&](int buf, int t, int j, i32x8_t& out) __attribute__((always_inline)) {
      const uint8_t* a = lds + buf * XBYTES + (j * FM + lr) * XPITCH + t * 64 + h * 32;
      const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(a);
      const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(a + 16);
      out = __builtin_bit_cast(i32x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    auto barrier = [&]() __attribute__((always_inline)) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    };

    // One stage = 32 MFMA pairs (K-step t = g / 8, row fragment j = g % 8), each pair two MFMAs (the wave's two column
    // fragments).  Besides its MFMAs a pair issues the LDS read of the fragment two pairs ahead; pairs 4q .. 4q + 3 of
    // K-step t also write piece 4t + q of the next stage's activations to LDS and refill its registers; pairs 4 and 5 of
    // a K-step refill the weight registers of the K-step before it.
    auto stage = [&](auto par_c, int c) __attribute__((always_inline)) {
      constexpr int PAR = decltype(par_c)::value;
      static_for<0, 32>([&](auto g_c) __attribute__((always_inline)) {
        constexpr int g = decltype(g_c)::value;
        constexpr int t = g / 8, j = g % 8;
        auto& a0 = j < 4 ? acc_lo[0][j % 4] : acc_hi[0][j % 4];
        auto& a1 = j < 4 ? acc_lo[1][j % 4] : acc_hi[1][j % 4];
        a0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wreg[0][t], xf[g % RING], a0, 0, 0, 0, 0, 0, 0);
        if constexpr (g == 30) barrier();
        // fragment of pair g + 2
        if constexpr (g + 2 < 32)
          read_xf(PAR, (g + 2) / 8, (g + 2) % 8, xf[(g + 2) % RING]);
        else
          read_xf(PAR ^ 1, 0, g + 2 - 32, xf[(g + 2) % RING]);
        __builtin_amdgcn_sched_barrier(0);
        a1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wreg[1][t], xf[g % RING], a1, 0, 0, 0, 0, 0, 0);
        if constexpr (j < 4) {
          constexpr int piece = 4 * t + j;
          store_x_piece(piece, PAR ^ 1);
          load_x_piece(piece, c + 2);
        } else if constexpr (j < 6) {
          // the K-step before this one has issued its last MFMA: its weight registers take the next use's data
          constexpr int tw = (t + NS - 1) % NS;
          load_w(j - 4, tw, t == 0 ? c : c + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    // Prologue: stage 0's activations to LDS, stage 1's into the staging registers, weights of K-steps 0..2 of stage 0
    // (K-step 3 is requested by stage 0 itself); the loads left in flight are in the order the steady state leaves them in.
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { store_x_piece(decltype(jc)::value, 0); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NS - 1>([&](auto tc) __attribute__((always_inline)) {
      load_w(0, decltype(tc)::value, 0);
      load_w(1, decltype(tc)::value, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, XCH>([&](auto jc) __attribute__((always_inline)) { load_x_piece(decltype(jc)::value, 1); });
    __builtin_amdgcn_sched_barrier(0);
    barrier();
    read_xf(0, 0, 0, xf[0]);
    read_xf(0, 0, 1, xf[1]);
    __builtin_amdgcn_sched_barrier(0);
    int c = 0;
    for (; c + 1 < nst; c += 2) {
      stage(template_int<0>{}, c);
      stage(template_int<1>{}, c + 1);
    }
    if (c < nst) stage(template_int<0>{}, c);
    // (the LDS reads behind the last stage's barrier fetch operands of a stage that does not exist and are not used; the
    // next tile's first LDS writes come behind its own loads and this tile's epilogue)
    barrier();
    gemm_epilogue<FM, 1, MFW / 2, NFW, SWIGLU>(p, acc_lo, expert, blk_off, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                               pid_n * BN + BN <= N, 0, lr, h);
    if (blk_rows > 128)
      gemm_epilogue<FM, 1, MFW / 2, NFW, SWIGLU>(p, acc_hi, expert, blk_off + 128, start_m, blk_off + blk_rows, pid_n * BN + nw * NFW * FM,
                                                 pid_n * BN + BN <= N, 0, lr, h);
  }  // tiles
}

}  // namespace

int32_t gemm_launch_f8w(const GemmParams& p, int grid_m, bool swiglu, hipStream_t st) {
  constexpr int LDS_BYTES = 2 * 256 * (256 + 16);
  GemmParams q = p;
  q.grid_n = (int)cdiv(p.N, 256);
  int64_t grid = (int64_t)grid_m * q.grid_n;
  if (grid <= 0) return TK_OK;
  if (grid > 0x7FFFFFFF) return fail(TK_ERR_UNSUPPORTED, "tk_moe_gemm: grid too large");
  q.total_tiles = (int32_t)grid;
  const int64_t resident = (int64_t)busy_cu_count(p.idle_cus);  // persistent grid, one workgroup per CU
  if (grid > resident) grid = resident;
  auto launch = [&](auto kern) -> int32_t {
    if (const int32_t rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), LDS_BYTES, st, q);
    return check_launch("moe_gemm_f8w_kernel");
  };
  if (swiglu) return launch(moe_gemm_f8w_kernel<true>);
  return launch(moe_gemm_f8w_kernel<false>);
}

}  // namespace tk
